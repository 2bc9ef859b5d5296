// Where a key or a value sits in its page. Pages hold page_size positions (a multiple of 16) of every kv head,
// in tiles of 16 positions laid out the way the MFMA kernels read them, so that a wave's load of a tile is one
// contiguous piece of memory:
//   keys:   [page][kv_head][tile][dim / 8][position % 16][dim % 8]
//           (lane (position, quad) of a wave reads 8 dims = 16 bytes of chunk 4 * k_step + quad)
//   values: [page][kv_head][tile][dim / 32][(position % 16) / 8][dim % 32][position % 8]
//           (lane (dim, half) of a wave reads the 8 positions 8 * half .. + 7 = 16 bytes for bfloat16, the 8
//           k-slots it supplies to one product, and the 64 lanes of a wave read 1024 consecutive bytes, which
//           LDS gives without bank conflicts; the keys' rows are taken in the order that makes the scores come
//           out so. A last block of 16 dims, where head_dim is an odd multiple of 16, is [position / 8][16][8].)
// head_dim is padded to a multiple of 8 (keys) or 16 (values); the padding is never read as data.
#pragma once

#include <stdint.h>

namespace mll {

struct CacheLayout {
    int kv_heads;
    int page_size;   // multiple of 16
    int head_dim;
    int tiles;       // page_size / 16
    int k_chunks;    // ceil(head_dim / 8)
    int v_dim_tiles; // ceil(head_dim / 16)

    __host__ __device__ CacheLayout(int kv_heads_, int page_size_, int head_dim_)
        : kv_heads(kv_heads_), page_size(page_size_), head_dim(head_dim_), tiles(page_size_ / 16),
          k_chunks((head_dim_ + 7) / 8), v_dim_tiles((head_dim_ + 15) / 16) {}

    // First element of a 16-position tile of keys / values.
    __host__ __device__ int64_t k_tile(int64_t page, int kv_head, int tile) const {
        return ((page * kv_heads + kv_head) * tiles + tile) * static_cast<int64_t>(k_chunks) * 128;
    }
    __host__ __device__ int64_t v_tile(int64_t page, int kv_head, int tile) const {
        return ((page * kv_heads + kv_head) * tiles + tile) * static_cast<int64_t>(v_dim_tiles) * 256;
    }
    // Element offsets inside a tile.
    __host__ __device__ static int k_in_tile(int position16, int dim) { return ((dim / 8) * 16 + position16) * 8 + dim % 8; }
    __host__ __device__ int v_in_tile(int position16, int dim) const {
        const int block = dim / 32;
        const int width = min_int(32, v_dim_tiles * 16 - 32 * block);      // dims of this block: 32, or 16 in a last half block
        return block * 512 + ((position16 / 8) * width + dim % 32) * 8 + position16 % 8;
    }
    __host__ __device__ static int min_int(int a, int b) { return a < b ? a : b; }
    __host__ __device__ int64_t k_at(int64_t page, int kv_head, int offset, int dim) const {
        return k_tile(page, kv_head, offset / 16) + k_in_tile(offset % 16, dim);
    }
    __host__ __device__ int64_t v_at(int64_t page, int kv_head, int offset, int dim) const {
        return v_tile(page, kv_head, offset / 16) + v_in_tile(offset % 16, dim);
    }
};

}  // namespace mll
