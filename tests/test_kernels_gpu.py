"""Each HIP kernel alone against a plain reference, at sizes other than the engine's tiny models use:
widths and vocabularies that are no powers of two, head sizes in steps of 16 (and, for the plain-path
kernel, one that is not), several group sizes, pages in a shuffled order."""
import math

import numpy as np
import pytest
import torch

import plain_qwen2 as plain

from microllm_rocm_amd.cache.layout import (key_page_shape, key_rows, value_page_shape, value_rows, write_key_rows,
                                            write_value_rows)

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"


def kernels():
    from microllm_rocm_amd.ops import kernels as module
    return module


def to_bf16_exact(array):
    """Round to bfloat16 and return (float64 numpy of the rounded values, bfloat16 tensor on the GPU)."""
    tensor = torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)
    return tensor.to(torch.float64).numpy(), tensor.to(DEVICE)


def prepare(array, dtype):
    if dtype == torch.bfloat16:
        return to_bf16_exact(array)
    value = np.asarray(array, dtype=np.float32)
    return value.astype(np.float64), torch.from_numpy(value).to(DEVICE)


def tolerance(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.2e-2, atol=1.2e-2)


# ---- embedding ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding(dtype):
    rng = np.random.default_rng(0)
    reference, table = prepare(rng.normal(size=(331, 100)), dtype)
    ids = np.array([5, 330, 0, 17, 5], dtype=np.int32)
    out = kernels().embedding(table, torch.from_numpy(ids).to(DEVICE))
    assert out.dtype == torch.float32
    np.testing.assert_array_equal(out.cpu().numpy().astype(np.float64), plain.embedding(reference, ids))
    bad = kernels().embedding(table, torch.tensor([3, 331, -1], dtype=torch.int32, device=DEVICE)).cpu()
    assert torch.isfinite(bad[0]).all() and torch.isnan(bad[1]).all() and torch.isnan(bad[2]).all()


# ---- norm ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("width", [24, 1000, 3584])
@pytest.mark.parametrize("out_dtype,delta_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32),
                                                   (torch.bfloat16, torch.bfloat16)])
def test_rms_norm_with_the_residual_sum(width, out_dtype, delta_dtype):
    rng = np.random.default_rng(width)
    h_ref = rng.normal(size=(7, width)).astype(np.float32)
    delta_ref, delta = prepare(rng.normal(size=(7, width)), delta_dtype)
    weight = (1 + 0.1 * rng.normal(size=width)).astype(np.float32)
    eps = 3e-4
    w = torch.from_numpy(weight).to(DEVICE)
    k = kernels()
    # plain
    h = torch.from_numpy(h_ref.copy()).to(DEVICE)
    out = k.rms_norm(h, w, eps, out_dtype)
    np.testing.assert_allclose(out.float().cpu().numpy(), plain.rms_norm(h_ref.astype(np.float64), weight, eps),
                               **tolerance(out_dtype))
    assert torch.equal(h.cpu(), torch.from_numpy(h_ref))
    # with the sum written back
    out = k.rms_norm(h, w, eps, out_dtype, delta=delta, write_h=True)
    total = h_ref.astype(np.float64) + delta_ref
    np.testing.assert_allclose(h.cpu().numpy(), total, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(out.float().cpu().numpy(), plain.rms_norm(total, weight, eps), **tolerance(out_dtype))
    # selected rows, nothing written
    h = torch.from_numpy(h_ref.copy()).to(DEVICE)
    rows = torch.tensor([6, 2, 2], dtype=torch.int32, device=DEVICE)
    out = k.rms_norm(h, w, eps, out_dtype, delta=delta, rows=rows)
    np.testing.assert_allclose(out.float().cpu().numpy(), plain.rms_norm(total[[6, 2, 2]], weight, eps), **tolerance(out_dtype))
    assert torch.equal(h.cpu(), torch.from_numpy(h_ref))
    k.residual_add(h, delta)
    np.testing.assert_allclose(h.cpu().numpy(), total, rtol=1e-6, atol=1e-6)


def test_rms_norm_vector_of_the_reference():
    # tests/ops/ops_test.cpp:480-485
    h = torch.tensor([[3.0, 4.0]], device=DEVICE)
    out = kernels().rms_norm(h, torch.tensor([1.0, 2.0], device=DEVICE), 1e-5, torch.float32).cpu().numpy()
    denominator = math.sqrt(12.5 + 1e-5)
    np.testing.assert_allclose(out, [[3 / denominator, 8 / denominator]], rtol=1e-6)


# ---- projections: bias, rotation, pages ----------------------------------------------------------------
def reference_qkv(qkv, bias, positions, theta, heads, kv_heads, hd, rotary):
    tokens = qkv.shape[0]
    x = qkv + (bias if bias is not None else 0.0)
    x = x.reshape(tokens, heads + 2 * kv_heads, hd)
    out = x.copy()
    if rotary:
        rotated = plain.rope_split_half(x[:, :heads + kv_heads, :rotary], positions, theta)
        out[:, :heads + kv_heads, :rotary] = rotated
    return out[:, :heads], out[:, heads:heads + kv_heads], out[:, heads + kv_heads:]


@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                                (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("heads,kv_heads,hd,rotary,page_size,use_bias", [
    (5, 5, 48, 48, 16, True), (6, 2, 16, 16, 48, False), (7, 1, 80, 32, 32, True), (3, 3, 24, 0, 16, True)])
def test_qkv_rope_store(in_dtype, out_dtype, heads, kv_heads, hd, rotary, page_size, use_bias):
    rng = np.random.default_rng(heads * 100 + hd)
    tokens, pages = 11, 9
    theta = 5e4
    qkv_ref, qkv = prepare(rng.normal(size=(tokens, (heads + 2 * kv_heads) * hd)), in_dtype)
    bias_ref = rng.normal(size=(heads + 2 * kv_heads) * hd).astype(np.float32) if use_bias else None
    positions = rng.integers(0, 3000, size=tokens).astype(np.int32)
    slots = rng.permutation(pages * page_size)[:tokens].astype(np.int32)
    slots[3] = -1
    inv_freq = None
    if rotary:
        inv_freq = torch.tensor(theta ** (-np.arange(0, rotary, 2, dtype=np.float64) / rotary), dtype=torch.float64, device=DEVICE)
    k_pages = torch.full(key_page_shape(pages, kv_heads, page_size, hd), 7.0, dtype=out_dtype, device=DEVICE)
    v_pages = torch.full(value_page_shape(pages, kv_heads, page_size, hd), 7.0, dtype=out_dtype, device=DEVICE)
    q = kernels().qkv_rope_store(qkv, torch.from_numpy(bias_ref).to(DEVICE) if use_bias else None,
                                 torch.from_numpy(positions).to(DEVICE), torch.from_numpy(slots).to(DEVICE), inv_freq,
                                 k_pages, v_pages, heads, kv_heads, hd, page_size, out_dtype)
    q_ref, k_ref, v_ref = reference_qkv(qkv_ref, None if bias_ref is None else bias_ref.astype(np.float64), positions,
                                        theta, heads, kv_heads, hd, rotary)
    tol = tolerance(out_dtype)
    np.testing.assert_allclose(q.float().cpu().numpy().reshape(tokens, heads, hd), q_ref, **tol)
    k_host = key_rows(k_pages, hd).float().cpu().numpy()        # [page, kv_head, position, dim]
    v_host = value_rows(v_pages, hd).float().cpu().numpy()
    written = np.zeros((pages, page_size), dtype=bool)
    for token, slot in enumerate(slots):
        if slot < 0:
            continue
        page, offset = divmod(int(slot), page_size)
        written[page, offset] = True
        np.testing.assert_allclose(k_host[page, :, offset, :], k_ref[token], **tol)
        np.testing.assert_allclose(v_host[page, :, offset, :], v_ref[token], **tol)
    assert np.all(k_host.transpose(0, 2, 1, 3)[~written] == 7.0) and np.all(v_host.transpose(0, 2, 1, 3)[~written] == 7.0)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,hd,page_size,parts", [(5, 5, 48, 16, 1), (6, 2, 16, 48, 3), (28, 4, 128, 16, 1), (3, 0, 24, 16, 2)])
def test_qkv_rope_store_with_many_tokens_takes_the_same_values(out_dtype, heads, kv_heads, hd, page_size, parts):
    """Many tokens with a table of cos and sin take the 16-byte kernel: the same bits as the kernel that goes pair by pair."""
    rng = np.random.default_rng(heads + hd)
    tokens, pages = 150, 12
    total = (heads + 2 * kv_heads) * hd
    qkv = torch.from_numpy(rng.normal(size=(parts, tokens, total)).astype(np.float32)).to(DEVICE)
    qkv = qkv[0].contiguous() if parts == 1 else qkv
    bias = torch.from_numpy(rng.normal(size=total).astype(np.float32)).to(DEVICE)
    positions = torch.from_numpy(rng.integers(0, 30000, size=tokens).astype(np.int32)).to(DEVICE)
    slots_host = rng.permutation(pages * page_size)[:tokens].astype(np.int32)
    slots_host[5] = -1
    slots = torch.from_numpy(slots_host).to(DEVICE) if kv_heads else None
    inv_freq = torch.tensor(1e6 ** (-np.arange(0, hd, 2, dtype=np.float64) / hd), dtype=torch.float64, device=DEVICE)
    table = kernels().rope_table(positions, inv_freq)

    def run(**how):
        k_pages = torch.full(key_page_shape(pages, kv_heads, page_size, hd), 7.0, dtype=out_dtype, device=DEVICE) if kv_heads else None
        v_pages = torch.full(value_page_shape(pages, kv_heads, page_size, hd), 7.0, dtype=out_dtype, device=DEVICE) if kv_heads else None
        q = kernels().qkv_rope_store(qkv, bias, positions, slots, how.get("inv_freq"), k_pages, v_pages, heads, kv_heads, hd,
                                     page_size, out_dtype, cos_sin=how.get("cos_sin"))
        return q, k_pages, v_pages

    wide = run(cos_sin=table)
    narrow = run(inv_freq=inv_freq)
    assert torch.equal(wide[0], narrow[0])
    if kv_heads:
        assert torch.equal(wide[1], narrow[1]) and torch.equal(wide[2], narrow[2])


def test_rope_vector_of_the_reference_and_large_positions():
    # tests/ops/ops_test.cpp:505-515: {5,6,7,8} at p=1, hd=4, base 10000
    qkv = torch.tensor([[5.0, 6.0, 7.0, 8.0]], device=DEVICE)
    inv_freq = torch.tensor([1.0, 10000.0 ** -0.5], dtype=torch.float64, device=DEVICE)
    q = kernels().qkv_rope_store(qkv, None, torch.tensor([1], dtype=torch.int32, device=DEVICE), None, inv_freq,
                                 None, None, 1, 0, 4, 16, torch.float32).cpu().numpy()[0]
    assert q[0] == pytest.approx(5 * math.cos(1.0) - 7 * math.sin(1.0), rel=1e-6)
    assert q[2] == pytest.approx(5 * math.sin(1.0) + 7 * math.cos(1.0), rel=1e-6)
    # the angle is exact in float64 before cos and sin are rounded: no drift at a position of 100 000
    q = kernels().qkv_rope_store(torch.tensor([[1.0, 0.0, 0.0, 0.0]], device=DEVICE), None,
                                 torch.tensor([100000], dtype=torch.int32, device=DEVICE), None, inv_freq, None, None,
                                 1, 0, 4, 16, torch.float32).cpu().numpy()[0]
    assert q[0] == pytest.approx(math.cos(100000.0), abs=1e-7) and q[2] == pytest.approx(math.sin(100000.0), abs=1e-7)


# ---- attention over pages ---------------------------------------------------------------------------------
def build_paged_case(rng, dtype, seq_lengths, counts, heads, kv_heads, hd, page_size, spare_pages=3):
    """Requests with ``seq_lengths`` cached positions in total, the last ``counts`` of them being this step's
    queries. Pages are assigned in a shuffled order; unused slots hold large finite garbage."""
    n_seqs = len(seq_lengths)
    blocks = [-(-length // page_size) for length in seq_lengths]
    total_pages = sum(blocks) + spare_pages
    order = rng.permutation(total_pages)
    width = max(blocks) + 1
    table = np.full((n_seqs, width), -1, dtype=np.int32)
    cursor = 0
    for s, count in enumerate(blocks):
        table[s, :count] = order[cursor:cursor + count]
        cursor += count
    k_ref = [rng.normal(size=(length, kv_heads, hd)) for length in seq_lengths]
    v_ref = [rng.normal(size=(length, kv_heads, hd)) for length in seq_lengths]
    k_rows = np.full((total_pages, kv_heads, page_size, hd), 1e4, dtype=np.float32)    # [page, kv_head, position, dim]
    v_rows = np.full((total_pages, kv_heads, page_size, hd), -1e4, dtype=np.float32)
    exact_k, exact_v = [], []
    for s, length in enumerate(seq_lengths):
        k_exact, _ = prepare(k_ref[s], dtype)
        v_exact, _ = prepare(v_ref[s], dtype)
        exact_k.append(k_exact)
        exact_v.append(v_exact)
        for position in range(length):
            page, offset = table[s, position // page_size], position % page_size
            k_rows[page, :, offset, :] = k_exact[position]
            v_rows[page, :, offset, :] = v_exact[position]
    k_pages = torch.zeros(key_page_shape(total_pages, kv_heads, page_size, hd), dtype=dtype, device=DEVICE)
    v_pages = torch.zeros(value_page_shape(total_pages, kv_heads, page_size, hd), dtype=dtype, device=DEVICE)
    write_key_rows(k_pages, torch.from_numpy(k_rows).to(dtype).to(DEVICE))
    write_value_rows(v_pages, torch.from_numpy(v_rows).to(dtype).to(DEVICE))
    seq_of_token = np.repeat(np.arange(n_seqs), counts).astype(np.int32)
    positions = np.concatenate([np.arange(length - count, length) for length, count in zip(seq_lengths, counts)]).astype(np.int32)
    q_exact, q = prepare(rng.normal(size=(len(positions), heads * hd)), dtype)
    tensors = dict(q=q, k=k_pages, v=v_pages,
                   table=torch.from_numpy(table).to(DEVICE), seq=torch.from_numpy(seq_of_token).to(DEVICE),
                   pos=torch.from_numpy(positions).to(DEVICE))
    return tensors, q_exact, exact_k, exact_v, seq_of_token, positions


def reference_attention(q_exact, exact_k, exact_v, seq_of_token, positions, heads, kv_heads, hd, scale, window):
    out = np.zeros((len(positions), heads, hd))
    group = heads // kv_heads
    for token, (s, p) in enumerate(zip(seq_of_token, positions)):
        low = 0 if not window else max(0, p - window + 1)
        for head in range(heads):
            keys = exact_k[s][low:p + 1, head // group]
            scores = keys @ q_exact[token].reshape(heads, hd)[head] * scale
            weights = np.exp(scores - scores.max())
            out[token, head] = (weights / weights.sum()) @ exact_v[s][low:p + 1, head // group]
    return out.reshape(len(positions), heads * hd)


def query_tile_list(lengths, counts):
    """(request, first token in the flat list, tokens, position of the first token) of every tile of 128 tokens."""
    tiles, start = [], 0
    for index, (length, count) in enumerate(zip(lengths, counts)):
        tiles += [(index, start + offset, min(128, count - offset), length - count + offset) for offset in range(0, count, 128)]
        start += count
    return tiles


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,hd,page_size,window", [
    (4, 2, 16, 16, 0), (3, 1, 32, 16, 24), (5, 5, 48, 16, 100), (6, 3, 24, 48, 0), (2, 1, 128, 32, 70), (8, 1, 200, 16, 0)])
def test_rowwise_attention(dtype, heads, kv_heads, hd, page_size, window):
    rng = np.random.default_rng(hd + window)
    lengths, counts = [150, 1, 64, 97], [40, 1, 64, 1]
    t, q_exact, ek, ev, seq, pos = build_paged_case(rng, dtype, lengths, counts, heads, kv_heads, hd, page_size)
    scale = 0.9 / math.sqrt(hd)
    out = kernels().paged_attention_rowwise(t["q"], t["k"], t["v"], t["table"], t["seq"], t["pos"], scale, window,
                                            heads, kv_heads, hd)
    reference = reference_attention(q_exact, ek, ev, seq, pos, heads, kv_heads, hd, scale, window)
    np.testing.assert_allclose(out.float().cpu().numpy(), reference, **tolerance(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,hd,page_size,window", [
    (4, 2, 16, 16, 0), (3, 1, 40, 16, 130), (6, 3, 128, 32, 0), (2, 1, 72, 16, 257), (5, 5, 48, 48, 1), (2, 2, 24, 16, 128),
    (28, 4, 128, 16, 0), (12, 2, 64, 16, 200), (10, 2, 32, 48, 0), (16, 1, 96, 16, 129), (9, 1, 16, 16, 0)])
def test_rowwise_attention_a_wave_per_chunk_gives_the_same_bits(dtype, heads, kv_heads, hd, page_size, window):
    """The plain kernel walks a row's keys by one wave, or by a wave per chunk of 128 keys with a merge: the same
    result to the last bit, whatever the row's position (chunk edges, one key beyond, many chunks) and window,
    and right against the reference. What the block table could hold beyond the longest request is no key."""
    rng = np.random.default_rng(hd * 3 + window)
    lengths, counts = [700, 1, 128, 129, 257, 384, 127], [130, 1, 2, 3, 1, 129, 1]
    t, q_exact, ek, ev, seq, pos = build_paged_case(rng, dtype, lengths, counts, heads, kv_heads, hd, page_size)
    scale = 0.9 / math.sqrt(hd)
    k = kernels()
    chunk = k.library.load().mll_paged_attention_rowwise_chunk()
    assert chunk == 128
    args = (t["q"], t["k"], t["v"], t["table"], t["seq"], t["pos"], scale, window, heads, kv_heads, hd)
    whole = k.paged_attention_rowwise(*args, split=False)
    by_chunk = k.paged_attention_rowwise(*args, split=True, longest=max(lengths))
    generous = k.paged_attention_rowwise(*args, split=True)      # as many chunks as the table is wide
    assert torch.equal(whole, by_chunk) and torch.equal(whole, generous)
    # in float32 a wave may take several query heads of a kv head, the group's last wave fewer: every count, forced
    usual = k.rowwise_heads_a_wave(1)
    several_heads, one_head = [], []
    try:
        one_head = [k.paged_attention_rowwise(*args, split=True, longest=max(lengths)), k.paged_attention_rowwise(*args, split=False)]
        for count in range(2, 9):
            k.rowwise_heads_a_wave(count)
            several_heads += [k.paged_attention_rowwise(*args, split=True, longest=max(lengths)), k.paged_attention_rowwise(*args, split=False)]
    finally:
        k.rowwise_heads_a_wave(usual)
    assert all(torch.equal(whole, other) for other in several_heads + one_head)
    reference = reference_attention(q_exact, ek, ev, seq, pos, heads, kv_heads, hd, scale, window)
    np.testing.assert_allclose(whole.float().cpu().numpy(), reference, **tolerance(dtype))
    assert k.rowwise_chunks(700, 0) == 6 and k.rowwise_chunks(128, 0) == 1 and k.rowwise_chunks(129, 0) == 2
    assert k.rowwise_chunks(5000, 1) == 1 and k.rowwise_chunks(5000, 2) == 2 and k.rowwise_chunks(5000, 129) == 2
    assert k.rowwise_chunks(5000, 130) == 3 and k.rowwise_chunks(100, 130) == 1


@pytest.mark.parametrize("heads,kv_heads,hd,page_size,window,splits", [
    (4, 2, 16, 16, 0, 1), (3, 1, 32, 16, 24, 2), (5, 5, 48, 16, 100, 3), (28, 4, 128, 16, 0, 8), (14, 2, 64, 32, 0, 5),
    (16, 1, 80, 16, 300, 4), (20, 1, 16, 48, 0, 2), (2, 2, 256, 16, 0, 7), (7, 7, 112, 64, 129, 1), (6, 3, 96, 16, 0, 64)])
def test_decode_attention(heads, kv_heads, hd, page_size, window, splits):
    rng = np.random.default_rng(heads + hd + splits)
    lengths = [517, 1, 33, 960, 16, 32, 129]
    t, q_exact, ek, ev, seq, pos = build_paged_case(rng, torch.bfloat16, lengths, [1] * len(lengths), heads, kv_heads, hd, page_size)
    scale = 1.0 / math.sqrt(hd)
    out = kernels().paged_attention_decode(t["q"], t["k"], t["v"], t["table"], t["seq"], t["pos"], scale, window,
                                           heads, kv_heads, hd, splits)
    reference = reference_attention(q_exact, ek, ev, seq, pos, heads, kv_heads, hd, scale, window)
    np.testing.assert_allclose(out.float().cpu().numpy(), reference, **tolerance(torch.bfloat16))
    # some rows only: the others are left as they were
    some = torch.tensor([5, 0, 3], dtype=torch.int32, device=DEVICE)
    partial = torch.full_like(out, 7.0)
    kernels().paged_attention_decode(t["q"], t["k"], t["v"], t["table"], t["seq"], t["pos"], scale, window,
                                     heads, kv_heads, hd, splits, out=partial, token_ids=some)
    assert torch.equal(partial[[5, 0, 3]], out[[5, 0, 3]]) and bool((partial[[1, 2, 4, 6]] == 7.0).all())


@pytest.mark.parametrize("heads,kv_heads,hd,page_size,window", [
    (4, 2, 16, 16, 0), (3, 1, 32, 16, 24), (5, 5, 48, 16, 100), (28, 4, 128, 16, 0), (14, 2, 64, 32, 40),
    (2, 1, 80, 16, 300), (3, 3, 256, 16, 0), (7, 7, 112, 64, 129), (6, 3, 96, 48, 17)])
def test_prefill_attention(heads, kv_heads, hd, page_size, window):
    rng = np.random.default_rng(heads + hd + window)
    lengths, counts = [517, 1, 700, 97, 64, 131, 40], [130, 1, 700, 17, 64, 2, 33]
    t, q_exact, ek, ev, seq, pos = build_paged_case(rng, torch.bfloat16, lengths, counts, heads, kv_heads, hd, page_size)
    scale = 1.0 / math.sqrt(hd)
    reference = reference_attention(q_exact, ek, ev, seq, pos, heads, kv_heads, hd, scale, window)
    tiles = query_tile_list(lengths, counts)
    alone = [(tile[0], tile[1], tile[2], 0, 0) for tile in tiles]
    backwards = [(tile[0], 0, 0, tile[1], tile[2]) for tile in tiles]
    # every way of putting tiles together gives the same numbers: a late tile with an early one, neighbours, each
    # tile alone as the first or as the second of its workgroup
    results = []
    for pairs in (kernels().pair_query_tiles(tiles), kernels().pair_query_tiles(tiles, adjacent=True), alone, backwards):
        query_tiles = torch.tensor(pairs, dtype=torch.int32, device=DEVICE)
        out = kernels().paged_attention_prefill(t["q"], t["k"], t["v"], t["table"], query_tiles, t["pos"], scale, window,
                                                heads, kv_heads, hd)
        np.testing.assert_allclose(out.float().cpu().numpy(), reference, **tolerance(torch.bfloat16))
        results.append(out)
    for out in results[1:]:
        assert torch.equal(out, results[0]), "a token's result depends on which tile shares its workgroup"


@pytest.mark.parametrize("kernel", ["rowwise_f32", "rowwise_bf16", "decode", "prefill"])
def test_a_far_key_among_hundreds_and_the_window_edge(kernel):
    """One key is made to dominate the softmax; the output must be that key's value. With random keys a wrong
    page or an off-by-one at the window's edge would change the result too little to see."""
    dtype = torch.float32 if kernel == "rowwise_f32" else torch.bfloat16
    heads, kv_heads, hd, page_size = 4, 2, 32, 16
    rng = np.random.default_rng(5)
    length = 700
    k = kernels()

    def run(target, window):
        t, q_exact, ek, ev, seq, pos = build_paged_case(rng, dtype, [length], [1], heads, kv_heads, hd, page_size)
        direction = rng.normal(size=hd)
        direction /= np.linalg.norm(direction)
        q = np.tile(direction * 16.0, heads)[None, :]
        table = t["table"].cpu().numpy()
        k_rows = key_rows(t["k"], hd).float()
        page, offset = table[0, target // page_size], target % page_size
        k_rows[page, :, offset, :] = torch.from_numpy(direction * 16.0).float()    # score 256 * scale against |others| ~ 16 * scale
        write_key_rows(t["k"], k_rows.to(dtype))
        _, t["q"] = prepare(q, dtype)
        scale = 1.0 / math.sqrt(hd)
        if kernel == "decode":
            out = k.paged_attention_decode(t["q"], t["k"], t["v"], t["table"], t["seq"], t["pos"], scale, window,
                                           heads, kv_heads, hd, 6)
        elif kernel == "prefill":
            out = k.paged_attention_prefill(t["q"], t["k"], t["v"], t["table"],
                                            torch.tensor([[0, 0, 1, 0, 0]], dtype=torch.int32, device=DEVICE), t["pos"],
                                            scale, window, heads, kv_heads, hd)
        else:
            out = k.paged_attention_rowwise(t["q"], t["k"], t["v"], t["table"], t["seq"], t["pos"], scale, window,
                                            heads, kv_heads, hd)
        return out.float().cpu().numpy().reshape(heads, hd), ev[0]

    for target in (3, 257, 688):
        out, values = run(target, 0)
        for head in range(heads):
            np.testing.assert_allclose(out[head], values[target, head // 2], atol=2e-2)
    window = 100                       # the query is at 699: keys 600..699 are visible
    out, values = run(600, window)     # the oldest visible key
    np.testing.assert_allclose(out[0], values[600, 0], atol=2e-2)
    out, values = run(599, window)     # one beyond the edge: it must not be seen
    assert np.abs(out[0] - values[599, 0]).max() > 0.3


# ---- feed-forward activation -------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [203, 208, 4864])
def test_silu_mul(dtype, width):
    rng = np.random.default_rng(1)
    reference, gate_up = prepare(np.concatenate([rng.normal(size=(9, 2 * width)) * 4, [[-90.0] * width + [1.0] * width]]), dtype)
    out = kernels().silu_mul(gate_up)
    expected = plain.silu(reference[:, :width]) * reference[:, width:]
    np.testing.assert_allclose(out.float().cpu().numpy(), expected, **tolerance(dtype))
    vector = kernels().silu_mul(torch.tensor([[-1.0, 0.0, 1.0, 2.0, 2.0, 2.0]], device=DEVICE)).cpu().numpy()[0]
    np.testing.assert_allclose(vector, [-2 / (1 + math.e), 0.0, 2 / (1 + math.exp(-1))], rtol=1e-6)   # ops_test.cpp:487-495


# ---- matrix products ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("m,n,k", [(1, 331, 120), (7, 64, 17), (65, 129, 200), (130, 1000, 96)])
def test_gemm_f32_and_row_independence(m, n, k):
    rng = np.random.default_rng(m)
    a, w, bias = rng.normal(size=(m, k)).astype(np.float32), rng.normal(size=(n, k)).astype(np.float32), rng.normal(size=n).astype(np.float32)
    ka = kernels()
    out = ka.gemm_f32(torch.from_numpy(a).to(DEVICE), torch.from_numpy(w).to(DEVICE), torch.from_numpy(bias).to(DEVICE))
    np.testing.assert_allclose(out.cpu().numpy(), a.astype(np.float64) @ w.astype(np.float64).T + bias, rtol=2e-5, atol=2e-5)
    # a row's result is bit-equal whatever other rows the call holds
    alone = ka.gemm_f32(torch.from_numpy(a[-1:]).to(DEVICE), torch.from_numpy(w).to(DEVICE), torch.from_numpy(bias).to(DEVICE))
    assert torch.equal(alone[0], out[-1])


@pytest.mark.parametrize("n,k,parts", [(3584, 3584, 8), (1152, 1792, 4), (896, 4864, 8), (37888, 512, 1), (640, 901, 2), (3000, 1026, 2), (200, 300, 1)])
def test_gemm_f32_in_parts_gives_every_row_the_same_bits_in_every_batch(n, k, parts):
    """The 32-bit product cuts the reduction of a weight with few rows of its own into parts by the weight's shape
    alone; the parts, added in order, are the product, and a row's parts are the same bits whether it comes alone, with
    15 others (one element a thread, or 2 x 2), with 40 (tiles of 16 x 32 or 32 x 64), 64 (64 x 64) or 600 (128 x 64):
    every kernel sums an element in ascending k with one fused multiply-add a term. Reductions that are no multiple of 4
    (no 16-byte loads) and of 2 mod 4 are among the shapes."""
    ka = kernels()
    assert ka.f32_splits(n, k) == parts
    rng = np.random.default_rng(n + k)
    a = rng.normal(size=(600, k)).astype(np.float32)
    w = (rng.normal(size=(n, k)) * 0.05).astype(np.float32)
    bias = rng.normal(size=n).astype(np.float32)
    device_a, device_w, device_bias = (torch.from_numpy(x).to(DEVICE) for x in (a, w, bias))
    whole = ka.gemm_f32(device_a, device_w, device_bias, partials=True)
    assert tuple(whole.shape) == ((parts, 600, n) if parts > 1 else (600, n))
    total = whole.double().sum(0) if parts > 1 else whole.double()
    expected = a.astype(np.float64) @ w.astype(np.float64).T + bias
    np.testing.assert_allclose(total.cpu().numpy(), expected, rtol=3e-5, atol=3e-5 * np.abs(expected).max())
    if parts > 1:      # the bias is in the first part alone, and the parts are sums over consecutive ranges of k
        part_length = -(-(-(-k // parts)) // 4) * 4
        second = a[:3, part_length:2 * part_length].astype(np.float64) @ w[:, part_length:2 * part_length].astype(np.float64).T
        np.testing.assert_allclose(whole[1, :3].double().cpu().numpy(), second, rtol=3e-5, atol=3e-5 * np.abs(second).max())
    for rows in (1, 7, 8, 9, 16, 40, 64):
        fewer = ka.gemm_f32(device_a[:rows].contiguous(), device_w, device_bias, partials=True)
        assert torch.equal(fewer, whole[..., :rows, :]), f"{rows} rows: other bits than the same rows among 600"
    # up to 16 rows any of three kernels may take the product: the same bits
    usual = ka.f32_small_variant(0)
    try:
        for variant in (1, 2, 4):
            ka.f32_small_variant(variant)
            for rows in (1, 2, 3, 5, 8, 13, 16):
                forced = ka.gemm_f32(device_a[:rows].contiguous(), device_w, device_bias, partials=True)
                assert torch.equal(forced, whole[..., :rows, :]), f"{rows} rows, kernel {variant}"
    finally:
        ka.f32_small_variant(usual)
    unsplit = ka.gemm_f32(device_a[:40].contiguous(), device_w, device_bias)      # one sum an element when the caller wants no parts
    assert tuple(unsplit.shape) == (40, n)
    np.testing.assert_allclose(unsplit.cpu().numpy(), expected[:40], rtol=3e-5, atol=3e-5 * np.abs(expected).max())


@pytest.mark.parametrize("m", [1, 3, 8, 33, 64, 100])
@pytest.mark.parametrize("n,k", [(331, 120), (1000, 96), (256, 3584), (4608, 512)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16(m, n, k, out_dtype):
    rng = np.random.default_rng(m + n)
    a_ref, a = to_bf16_exact(rng.normal(size=(m, k)))
    w_ref, w = to_bf16_exact(rng.normal(size=(n, k)) * 0.1)
    out = kernels().gemm_bf16(a, w, out_dtype)
    assert out.dtype == out_dtype
    expected = a_ref @ w_ref.T
    scale = np.abs(expected).max()
    bound = 1e-5 if out_dtype == torch.float32 else 5e-3
    assert np.abs(out.float().cpu().numpy() - expected).max() <= bound * scale


# ---- selection ---------------------------------------------------------------------------------------------------
def test_argmax_rules():
    k = kernels()
    assert k.argmax(torch.tensor([[-2.0, 5.0, 5.0, 4.0]], device=DEVICE)).tolist() == [1]       # ops_test.cpp:414-439
    rows = torch.tensor([[1.0, 3.0, 2.0], [5.0, 5.0, 4.0], [1.0, float("inf"), 0.0], [float("nan"), 1.0, 2.0]], device=DEVICE)
    assert k.argmax(rows).tolist() == [1, 0, -1, -1]
    rng = np.random.default_rng(0)
    big = rng.normal(size=(5, 152064)).astype(np.float32)
    big[2, 77] = big[2, 150000] = 9.0
    assert k.argmax(torch.from_numpy(big).to(DEVICE)).tolist() == np.argmax(big, axis=1).tolist()
    assert k.argmax(torch.from_numpy(big[:, :331].copy()).to(DEVICE)).tolist() == np.argmax(big[:, :331], axis=1).tolist()


@pytest.mark.parametrize("vocab,top_k", [(331, 0), (331, 5), (5000, 50), (152064, 0), (152064, 40), (40, 40), (40, 39),
                                         (9001, 3000), (152064, 100000), (2049, 2)])
def test_sampling_follows_the_plain_rule(vocab, top_k):
    rng = np.random.default_rng(vocab + top_k)
    rows = 24
    logits = (rng.normal(size=(rows, vocab)) * 2).astype(np.float32)
    logits[0, 3] = logits[0, 9] = logits[0].max() + 1.0      # ties at the top
    logits[1, :] = np.round(logits[1, :])                    # many ties, also at the k-th value
    temperature = rng.choice([0.7, 1.0, 1.3], size=rows).astype(np.float32)
    temperature[2] = 0.0
    uniform = np.array([plain.uniform_for(5, draw) for draw in range(rows)], dtype=np.float32)
    chosen = kernels().sample(torch.from_numpy(logits).to(DEVICE), torch.from_numpy(temperature).to(DEVICE),
                              torch.full((rows,), top_k, dtype=torch.int32, device=DEVICE),
                              torch.from_numpy(uniform).to(DEVICE)).tolist()
    for row in range(rows):
        row_logits = logits[row].astype(np.float64)
        if temperature[row] == 0.0:
            assert chosen[row] == plain.greedy(row_logits)
            continue
        weights = plain.sampling_weights(row_logits, float(temperature[row]), top_k)
        assert weights[chosen[row]] > 0.0, "a token outside the top_k was drawn"
        cumulative = np.cumsum(weights)
        target = float(uniform[row]) * cumulative[-1]
        slack = 2e-4 * cumulative[-1]      # float32 sums on the device against float64 here
        low = cumulative[chosen[row]] - weights[chosen[row]]
        assert low - slack <= target <= cumulative[chosen[row]] + slack, f"row {row}: the draw is outside the token's interval"
    bad = logits.copy()
    bad[4, 100 % vocab] = np.nan
    out = kernels().sample(torch.from_numpy(bad).to(DEVICE), torch.from_numpy(temperature).to(DEVICE), None,
                           torch.from_numpy(uniform).to(DEVICE)).tolist()
    assert out[4] == -1 and all(token >= 0 for index, token in enumerate(out) if index != 4)


def test_sampling_with_a_rule_per_row_and_draws_at_both_ends():
    """Rows of one call differ in top_k and temperature; uniforms near 0 and near 1 fall into the first and the
    last selected tokens, which lie in different slices of the row."""
    rng = np.random.default_rng(11)
    vocab, rows = 50021, 12
    logits = (rng.normal(size=(rows, vocab)) * 1.5).astype(np.float32)
    top_k = np.array([0, 1, 7, 300, 0, 50020, 2, 0, 9, 9, 0, 1000], dtype=np.int32)
    temperature = np.array([0.9, 1.0, 1.1, 0.6, 0.0, 1.0, 0.8, 2.0, 0.7, 0.7, 1.0, 1.4], dtype=np.float32)
    uniform = np.array([0.0, 0.5, 0.999999, 0.0, 0.3, 0.999999, 0.5, 0.999999, 0.0, 0.999999, 1e-7, 0.25], dtype=np.float32)
    chosen = kernels().sample(torch.from_numpy(logits).to(DEVICE), torch.from_numpy(temperature).to(DEVICE),
                              torch.from_numpy(top_k).to(DEVICE), torch.from_numpy(uniform).to(DEVICE)).tolist()
    for row in range(rows):
        row_logits = logits[row].astype(np.float64)
        if temperature[row] == 0.0 or top_k[row] == 1:
            assert chosen[row] == plain.greedy(row_logits)
            continue
        weights = plain.sampling_weights(row_logits, float(temperature[row]), int(top_k[row]))
        assert weights[chosen[row]] > 0.0
        cumulative = np.cumsum(weights)
        target = float(uniform[row]) * cumulative[-1]
        slack = 2e-4 * cumulative[-1]
        assert cumulative[chosen[row]] - weights[chosen[row]] - slack <= target <= cumulative[chosen[row]] + slack, row
    selected = np.flatnonzero(plain.sampling_weights(logits[2].astype(np.float64), 1.1, 7))
    assert chosen[0] == 0 and chosen[2] == selected[-1] and chosen[8] == np.flatnonzero(
        plain.sampling_weights(logits[8].astype(np.float64), 0.7, 9))[0]


def test_sampling_frequencies():
    logits = torch.tensor([[1.0, 0.0, -1.0, 0.5, -30.0]], device=DEVICE).repeat(4000, 1)
    uniform = torch.tensor([plain.uniform_for(9, draw) for draw in range(4000)], dtype=torch.float32, device=DEVICE)
    chosen = kernels().sample(logits, torch.full((4000,), 0.8, device=DEVICE), None, uniform).cpu().numpy()
    expected = np.exp(np.array([1.0, 0.0, -1.0, 0.5, -30.0]) / 0.8)
    np.testing.assert_allclose(np.bincount(chosen, minlength=5) / 4000, expected / expected.sum(), atol=0.025)


# ---- the streaming product for few rows -------------------------------------------------------------------------
@pytest.mark.parametrize("m", [1, 5, 16, 17, 40, 64])
@pytest.mark.parametrize("n,k", [(331, 120), (96, 64), (1000, 200), (4608, 3584), (176, 24), (3584, 18944), (40000, 256)])
def test_gemm_skinny(m, n, k):
    rng = np.random.default_rng(m * 7 + n)
    a_ref, a = to_bf16_exact(rng.normal(size=(m, k)))
    w_ref, w = to_bf16_exact(rng.normal(size=(n, k)) * 0.1)
    ka = kernels()
    packed = ka.pack_weight(w)
    assert packed.shape == (-(-n // 16), -(-k // 32), 4, 16, 8)
    expected = a_ref @ w_ref.T
    scale = np.abs(expected).max()
    full = ka.gemm_skinny(a, packed, n, "f32")
    assert full.dtype == torch.float32 and full.shape == (m, n)
    assert np.abs(full.double().cpu().numpy() - expected).max() <= 1e-5 * scale
    out = ka.gemm_skinny(a, packed, n, "bf16")
    assert out.dtype == torch.bfloat16 and np.abs(out.float().cpu().numpy() - expected).max() <= 5e-3 * scale
    # the same in every run, and a row's result does not depend on the other rows of the call
    assert torch.equal(ka.gemm_skinny(a, packed, n, "f32"), full)
    alone = ka.gemm_skinny(a[m - 1:m].contiguous(), packed, n, "f32")
    assert torch.equal(alone[0], full[m - 1])


@pytest.mark.parametrize("m,width,k", [(3, 203, 96), (16, 176, 64), (33, 1000, 120)])
def test_gemm_skinny_gated_epilogue(m, width, k):
    rng = np.random.default_rng(width)
    a_ref, a = to_bf16_exact(rng.normal(size=(m, k)))
    w_ref, w = to_bf16_exact(rng.normal(size=(2 * width, k)) * 0.2)      # rows: [gate; up]
    packed = kernels().pack_weight(w, interleave_halves=True)
    out = kernels().gemm_skinny(a, packed, 2 * width, "gated")
    expected = plain.silu(a_ref @ w_ref[:width].T) * (a_ref @ w_ref[width:].T)
    assert out.shape == (m, width)
    np.testing.assert_allclose(out.float().cpu().numpy(), expected, rtol=1.2e-2, atol=1.2e-2 * np.abs(expected).max())


@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("heads,kv_heads,hd,rotary,hidden,bias", [(4, 2, 16, 16, 64, True), (3, 1, 32, 32, 96, True), (28, 4, 128, 128, 512, True),
                                                                   (5, 5, 48, 24, 40, False), (2, 0, 64, 64, 72, True)])
def test_gemm_skinny_qkv_is_product_then_rope_store(m, heads, kv_heads, hd, rotary, hidden, bias):
    """The fused epilogue against the two kernels it replaces: the product in float32, then bias, rotation and page write."""
    rng = np.random.default_rng(m + heads)
    ka = kernels()
    total = (heads + 2 * kv_heads) * hd
    _, x = to_bf16_exact(rng.normal(size=(m, hidden)))
    _, w = to_bf16_exact(rng.normal(size=(total, hidden)) * 0.2)
    b = torch.from_numpy(rng.normal(size=total).astype(np.float32)).to(DEVICE) if bias else None
    inv_freq = torch.from_numpy(1e4 ** -(np.arange(0, rotary, 2) / rotary)).to(DEVICE)
    positions = torch.from_numpy(rng.integers(0, 30000, size=m).astype(np.int32)).to(DEVICE)
    page_size, n_pages = 32, 6
    slots = torch.from_numpy(rng.permutation(page_size * n_pages)[:m].astype(np.int32)).to(DEVICE) if kv_heads else None

    def pages():
        if not kv_heads:
            return None, None
        from microllm_rocm_amd.cache.layout import key_page_shape, value_page_shape
        return (torch.zeros(key_page_shape(n_pages, kv_heads, page_size, hd), dtype=torch.bfloat16, device=DEVICE),
                torch.zeros(value_page_shape(n_pages, kv_heads, page_size, hd), dtype=torch.bfloat16, device=DEVICE))

    k_two, v_two = pages()
    q_two = ka.qkv_rope_store(ka.gemm_skinny(x, ka.pack_weight(w), total, "f32"), b, positions, slots, inv_freq, k_two, v_two,
                              heads, kv_heads, hd, page_size, torch.bfloat16)
    order = ka.rotary_pair_order(heads, kv_heads, hd, rotary // 2)
    assert sorted(order.tolist()) == list(range(total))
    packed = ka.pack_weight(w, row_order=order)
    k_one, v_one = pages()
    table = ka.rope_table(positions, inv_freq)
    angles = positions.cpu().numpy().astype(np.float64)[:, None] * inv_freq.cpu().numpy()[None, :]
    assert np.abs(table.cpu().numpy().astype(np.float64) - np.stack([np.cos(angles), np.sin(angles)], axis=-1)).max() <= 6e-8
    q_one = ka.gemm_skinny_qkv(x, packed, b, slots, table, k_one, v_one, heads, kv_heads, hd, page_size)
    assert torch.equal(q_one, q_two)
    if kv_heads:
        assert torch.equal(k_one, k_two) and torch.equal(v_one, v_two)
        assert k_one.float().abs().sum() > 0 and v_one.float().abs().sum() > 0
    # the unfused kernel reads products whose columns are in pair order
    k_three, v_three = pages()
    q_three = ka.qkv_rope_store(ka.gemm_skinny(x, packed, total, "f32"), b, positions, slots, None, k_three, v_three,
                                heads, kv_heads, hd, page_size, torch.bfloat16, pair_order=True, cos_sin=table)
    assert torch.equal(q_three, q_two)
    if kv_heads:
        assert torch.equal(k_three, k_two) and torch.equal(v_three, v_two)


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("n,k,n2", [(72, 320, 144), (3584, 512, 1024), (104, 96, 5000), (4096, 64, 96)])
def test_product_adds_to_the_stream_and_begins_the_norm(m, n, k, n2):
    """``gemm_skinny_residual`` then a product with the rows' factors, against sum, RMS norm and product done apart."""
    rng = np.random.default_rng(m + n)
    ka = kernels()
    x_ref, x = to_bf16_exact(rng.normal(size=(m, k)))
    w1_ref, w1 = to_bf16_exact(rng.normal(size=(n, k)) * 0.1)
    w2_ref, w2 = to_bf16_exact(rng.normal(size=(n2, n)) * 0.1)
    h_ref = rng.normal(size=(m, n)).astype(np.float32)
    norm_ref = (1.0 + 0.1 * rng.normal(size=n)).astype(np.float32)
    eps = 1e-5
    h = torch.from_numpy(h_ref.copy()).to(DEVICE)
    norm = torch.from_numpy(norm_ref).to(DEVICE)
    values, scale = ka.gemm_skinny_residual(x, ka.pack_weight(w1), h, norm, n, eps)
    total = h_ref.astype(np.float64) + x_ref @ w1_ref.T
    np.testing.assert_allclose(h.cpu().numpy(), total, rtol=1e-5, atol=1e-5 * np.abs(total).max())
    assert values.dtype == torch.bfloat16 and scale.sumsq.shape[0] == m and scale.width == n
    np.testing.assert_allclose(values.float().cpu().numpy(), total * norm_ref, rtol=8e-3, atol=1e-6)
    np.testing.assert_allclose(scale.sumsq[:, :scale.groups].double().sum(dim=1).cpu().numpy(), (total ** 2).sum(axis=1), rtol=1e-5)
    expected = plain.rms_norm(total, norm_ref, eps) @ w2_ref.T
    bound = 1.2e-2 * np.abs(expected).max()
    packed2 = ka.pack_weight(w2)
    out = ka.gemm_skinny(values, packed2, n2, "f32", scale=scale)
    assert np.abs(out.double().cpu().numpy() - expected).max() <= bound
    # the factors are the norm's: the same product of the norm's own output differs by rounding only
    h_two = torch.from_numpy(h_ref.copy()).to(DEVICE)
    normed = ka.rms_norm(h_two, norm, eps, torch.bfloat16, delta=ka.gemm_skinny(x, ka.pack_weight(w1), n, "f32"), write_h=True)
    apart = ka.gemm_skinny(normed, packed2, n2, "f32")
    assert np.abs(apart.double().cpu().numpy() - expected).max() <= bound
    assert torch.equal(h_two, h)
    # a row's result does not depend on the other rows
    h_one = torch.from_numpy(h_ref[m - 1:m].copy()).to(DEVICE)
    values_one, scale_one = ka.gemm_skinny_residual(x[m - 1:m].contiguous(), ka.pack_weight(w1), h_one, norm, n, eps)
    assert torch.equal(values_one[0], values[m - 1]) and torch.equal(h_one[0], h[m - 1])
    alone = ka.gemm_skinny(values_one, packed2, n2, "f32", scale=scale_one)
    assert torch.equal(alone[0], out[m - 1])


@pytest.mark.parametrize("m", [17, 33, 40, 64, 5])
@pytest.mark.parametrize("n,k", [(331, 120), (1000, 200), (4608, 3584), (176, 24), (3584, 18944), (40000, 256), (896, 4864)])
def test_gemm_medium(m, n, k):
    rng = np.random.default_rng(m * 11 + n)
    a_ref, a = to_bf16_exact(rng.normal(size=(m, k)))
    w_ref, w = to_bf16_exact(rng.normal(size=(n, k)) * 0.1)
    ka = kernels()
    packed = ka.pack_weight(w)
    expected = a_ref @ w_ref.T
    scale = np.abs(expected).max()
    parts = ka.gemm_medium(a, packed, n, "f32")                # its own plan: may split k
    tiles, waves, splits = ka.medium_plan(n, k)
    assert parts.dtype == torch.float32 and tuple(parts.shape) == ((splits, m, n) if splits > 1 else (m, n))
    total = parts.double().sum(dim=0) if splits > 1 else parts.double()
    assert np.abs(total.cpu().numpy() - expected).max() <= 1e-5 * scale
    whole = ka.gemm_medium(a, packed, n, "f32", plan=ka.medium_plan(n, k, may_split=False))
    assert tuple(whole.shape) == (m, n) and np.abs(whole.double().cpu().numpy() - expected).max() <= 1e-5 * scale
    out = ka.gemm_medium(a, packed, n, "bf16")
    assert out.dtype == torch.bfloat16 and np.abs(out.float().cpu().numpy() - expected).max() <= 5e-3 * scale
    # every plan the kernel takes gives the product
    for plan in ((1, 4, 1), (2, 4, 3), (2, 8, 2), (1, 8, 64)):
        other = ka.gemm_medium(a, packed, n, "f32", plan=plan)
        other = other.double().sum(dim=0) if other.dim() == 3 else other.double()
        assert np.abs(other.cpu().numpy() - expected).max() <= 1e-5 * scale, plan
    # the same in every run, and a row's result does not depend on the other rows of the call
    assert torch.equal(ka.gemm_medium(a, packed, n, "f32"), parts)
    alone = ka.gemm_medium(a[m - 1:m].contiguous(), packed, n, "f32")
    assert torch.equal(alone[..., 0, :], parts[..., m - 1, :])


@pytest.mark.parametrize("m,n,k,parts", [(300, 200, 4096, 2), (65, 331, 8192, 4), (700, 272, 16384, 8), (90, 64, 96, 3), (128, 256, 512, 1)])
def test_library_product_in_parts_of_the_reduction(m, n, k, parts):
    """The library's batched product over strided views: its parts add up to the whole product, each part is the
    product over its own range of the reduction."""
    rng = np.random.default_rng(m + k)
    a_ref, a = to_bf16_exact(rng.normal(size=(m, k)))
    w_ref, w = to_bf16_exact(rng.normal(size=(n, k)) * 0.1)
    ka = kernels()
    got = ka.gemm_bf16_split(a, w, parts)
    assert got.dtype == torch.float32 and got.shape == (parts, m, n)
    length = k // parts
    for part in range(parts):
        expected = a_ref[:, part * length:(part + 1) * length] @ w_ref[:, part * length:(part + 1) * length].T
        assert np.abs(got[part].double().cpu().numpy() - expected).max() <= 1e-5 * np.abs(expected).max()
    whole = a_ref @ w_ref.T
    assert np.abs(got.double().sum(0).cpu().numpy() - whole).max() <= 1e-5 * np.abs(whole).max()
    with pytest.raises(Exception, match="do not divide"):
        ka.gemm_bf16_split(a, w, 7)


@pytest.mark.parametrize("m,n,k", [(300, 1000, 256), (257, 272, 64), (65, 331, 96), (2048, 4608, 512), (700, 3584, 2048)])
def test_gemm_tiled(m, n, k):
    """The tiled product for many rows over a packed weight (what an engine with one copy of its weights takes)."""
    rng = np.random.default_rng(m + n)
    a_ref, a = to_bf16_exact(rng.normal(size=(m, k)))
    w_ref, w = to_bf16_exact(rng.normal(size=(n, k)) * 0.1)
    ka = kernels()
    packed = ka.pack_weight(w)
    expected = a_ref @ w_ref.T
    scale = np.abs(expected).max()
    full = ka.gemm_tiled(a, packed, n, "f32")
    assert full.dtype == torch.float32 and full.shape == (m, n)
    assert np.abs(full.double().cpu().numpy() - expected).max() <= 1e-5 * scale
    out = ka.gemm_tiled(a, packed, n, "bf16")
    assert out.dtype == torch.bfloat16 and np.abs(out.float().cpu().numpy() - expected).max() <= 5e-3 * scale
    if n % 2 == 0:
        gated = ka.gemm_tiled(a, ka.pack_weight(w, interleave_halves=True), n, "gated")
        wanted = plain.silu(expected[:, : n // 2]) * expected[:, n // 2:]
        np.testing.assert_allclose(gated.float().cpu().numpy(), wanted, rtol=1.2e-2, atol=1.2e-2 * np.abs(wanted).max())
    # the reduction in parts: the parts add up to the product, a part is the product over its stages of 64
    for splits in (2, 3, 8):
        parts = ka.gemm_tiled(a, packed, n, "f32", splits=splits)
        assert parts.shape == (splits, m, n)
        assert np.abs(parts.double().sum(0).cpu().numpy() - expected).max() <= 1e-5 * scale
        stages = -(-k // 64)
        per_part = -(-stages // splits)
        first = a_ref[:, :64 * per_part] @ w_ref[:, :64 * per_part].T
        assert np.abs(parts[0].double().cpu().numpy() - first).max() <= 1e-5 * max(np.abs(first).max(), 1e-30)
    with pytest.raises(Exception, match="parts"):
        ka.gemm_tiled(a, packed, n, "bf16", splits=2)
    # the same in every run, and a row's result does not depend on the other rows of the call
    assert torch.equal(ka.gemm_tiled(a, packed, n, "f32"), full)
    assert torch.equal(ka.gemm_tiled(a[m - 70:].contiguous(), packed, n, "f32"), full[m - 70:]) if m > 70 else True
    # nor on how many rows a workgroup's tile has
    assert ka.tiled_tile_rows(m, n) in (256, 192, 160, 128)
    for tile_rows in (256, 192, 160, 128):
        assert torch.equal(ka.gemm_tiled(a, packed, n, "f32", tile_rows=tile_rows), full), tile_rows
        assert torch.equal(ka.gemm_tiled(a, packed, n, "bf16", tile_rows=tile_rows), out), tile_rows
        assert torch.equal(ka.gemm_tiled(a, packed, n, "f32", splits=3, tile_rows=tile_rows), ka.gemm_tiled(a, packed, n, "f32", splits=3))
    with pytest.raises(Exception, match="256, 192, 160 or 128"):
        ka.gemm_tiled(a, packed, n, "f32", tile_rows=64)
    with pytest.raises(Exception, match="multiple of 32"):
        ka.gemm_tiled(a[:, :k - 8].contiguous(), ka.pack_weight(w[:, :k - 8].contiguous()), n)


@pytest.mark.parametrize("m", [65, 300, 600])
@pytest.mark.parametrize("heads,kv_heads,hd,rotary,hidden,bias", [(4, 2, 16, 16, 64, True), (3, 1, 32, 32, 96, True), (28, 4, 128, 128, 512, True),
                                                                   (5, 5, 48, 24, 160, False), (2, 0, 64, 64, 96, True), (7, 1, 80, 0, 32, True)])
def test_gemm_tiled_qkv_is_product_then_rope_store(m, heads, kv_heads, hd, rotary, hidden, bias):
    """The tiled product's q/k/v epilogue: against float64 numpy (bias, split-half rotation, pages read back), and
    the same bits as the two kernels it replaces. Rows past a tile's edge, slots of -1 and pages filled before
    show what is written where it should not be."""
    rng = np.random.default_rng(m + heads)
    ka = kernels()
    total = (heads + 2 * kv_heads) * hd
    theta = 1e4
    x_ref, x = to_bf16_exact(rng.normal(size=(m, hidden)))
    w_ref, w = to_bf16_exact(rng.normal(size=(total, hidden)) * 0.2)
    b_ref = rng.normal(size=total).astype(np.float32) if bias else None
    b = torch.from_numpy(b_ref).to(DEVICE) if bias else None
    inv_freq = torch.from_numpy(theta ** -(np.arange(0, rotary, 2) / rotary)).to(DEVICE) if rotary else None
    positions_host = rng.integers(0, 30000, size=m).astype(np.int32)
    positions = torch.from_numpy(positions_host).to(DEVICE)
    page_size = 32
    n_pages = -(-m // page_size) + 2
    slots_host = rng.permutation(page_size * n_pages)[:m].astype(np.int32)
    slots_host[[3, m - 1]] = -1
    slots = torch.from_numpy(slots_host).to(DEVICE) if kv_heads else None

    def pages():
        if not kv_heads:
            return None, None
        return (torch.full(key_page_shape(n_pages, kv_heads, page_size, hd), 7.0, dtype=torch.bfloat16, device=DEVICE),
                torch.full(value_page_shape(n_pages, kv_heads, page_size, hd), 7.0, dtype=torch.bfloat16, device=DEVICE))

    order = ka.rotary_pair_order(heads, kv_heads, hd, rotary // 2)
    packed = ka.pack_weight(w, row_order=order)
    table = ka.rope_table(positions, inv_freq) if rotary else None
    k_one, v_one = pages()
    q_one = ka.gemm_tiled_qkv(x, packed, b, slots, table, k_one, v_one, heads, kv_heads, hd, page_size)
    assert q_one.shape == (m, heads * hd) and q_one.dtype == torch.bfloat16

    q_ref, k_ref, v_ref = reference_qkv(x_ref @ w_ref.T, None if b_ref is None else b_ref.astype(np.float64), positions_host,
                                        theta, heads, kv_heads, hd, rotary)
    tol = dict(rtol=8e-3, atol=8e-3)
    np.testing.assert_allclose(q_one.float().cpu().numpy().reshape(m, heads, hd), q_ref, **tol)
    if kv_heads:
        k_host = key_rows(k_one, hd).float().cpu().numpy()        # [page, kv_head, position, dim]
        v_host = value_rows(v_one, hd).float().cpu().numpy()
        written = np.zeros((n_pages, page_size), dtype=bool)
        for token, slot in enumerate(slots_host):
            if slot < 0:
                continue
            page, offset = divmod(int(slot), page_size)
            written[page, offset] = True
            np.testing.assert_allclose(k_host[page, :, offset, :], k_ref[token], **tol)
            np.testing.assert_allclose(v_host[page, :, offset, :], v_ref[token], **tol)
        assert np.all(k_host.transpose(0, 2, 1, 3)[~written] == 7.0) and np.all(v_host.transpose(0, 2, 1, 3)[~written] == 7.0)

    k_two, v_two = pages()
    q_two = ka.qkv_rope_store(ka.gemm_tiled(x, packed, total, "f32"), b, positions, slots, None, k_two, v_two,
                              heads, kv_heads, hd, page_size, torch.bfloat16, pair_order=True, cos_sin=table)
    assert torch.equal(q_one, q_two)
    if kv_heads:
        assert torch.equal(k_one, k_two) and torch.equal(v_one, v_two)
    for tile_rows in (256, 192, 160, 128):
        k_three, v_three = pages()
        q_three = ka.gemm_tiled_qkv(x, packed, b, slots, table, k_three, v_three, heads, kv_heads, hd, page_size, tile_rows=tile_rows)
        assert torch.equal(q_three, q_one), tile_rows
        if kv_heads:
            assert torch.equal(k_three, k_one) and torch.equal(v_three, v_one), tile_rows


def test_tiles_of_fewer_rows_where_they_fill_the_compute_units():
    ka = kernels()
    assert ka.tiled_tile_rows(2048, 4608) == 160       # 144 tiles of 256 rows, 234 of 160
    assert ka.tiled_tile_rows(2048, 37888) == 256      # many rounds either way: the tile that loads least a product
    assert ka.tiled_tile_rows(2048, 3584, 2) == 256    # 224 workgroups in one round
    assert ka.tiled_tile_rows(100, 512) == 128         # one round whatever the height: the cheapest tile


def test_gemm_tiled_qkv_refuses_what_it_cannot_do():
    ka = kernels()
    x = torch.zeros((70, 40), dtype=torch.bfloat16, device=DEVICE)
    w = torch.zeros((2 * 16, 40), dtype=torch.bfloat16, device=DEVICE)
    with pytest.raises(Exception, match="k % 32"):
        ka.gemm_tiled_qkv(x, ka.pack_weight(w), None, None, None, None, None, 2, 0, 16, 16)
    x = torch.zeros((70, 64), dtype=torch.bfloat16, device=DEVICE)
    w = torch.zeros((2 * 48, 64), dtype=torch.bfloat16, device=DEVICE)
    odd = torch.zeros((70, 3, 2), dtype=torch.float32, device=DEVICE)       # three rotary pairs
    with pytest.raises(Exception, match="even number of rotary pairs"):
        ka.gemm_tiled_qkv(x, ka.pack_weight(w), None, None, odd, None, None, 2, 0, 48, 16)


@pytest.mark.parametrize("m,width,k", [(20, 203, 96), (64, 176, 64), (33, 1000, 520)])
def test_gemm_medium_gated_epilogue(m, width, k):
    rng = np.random.default_rng(width + 1)
    a_ref, a = to_bf16_exact(rng.normal(size=(m, k)))
    w_ref, w = to_bf16_exact(rng.normal(size=(2 * width, k)) * 0.2)      # rows: [gate; up]
    packed = kernels().pack_weight(w, interleave_halves=True)
    out = kernels().gemm_medium(a, packed, 2 * width, "gated")
    expected = plain.silu(a_ref @ w_ref[:width].T) * (a_ref @ w_ref[width:].T)
    assert out.shape == (m, width)
    np.testing.assert_allclose(out.float().cpu().numpy(), expected, rtol=1.2e-2, atol=1.2e-2 * np.abs(expected).max())


def test_gemm_medium_refuses_what_it_cannot_do():
    ka = kernels()
    a = torch.zeros((65, 64), dtype=torch.bfloat16, device=DEVICE)
    packed = ka.pack_weight(torch.zeros((32, 64), dtype=torch.bfloat16, device=DEVICE))
    with pytest.raises(Exception, match="at most 64 rows"):
        ka.gemm_medium(a, packed, 32)
    with pytest.raises(Exception, match="split"):
        ka.gemm_medium(a[:20], packed, 32, "bf16", plan=(1, 8, 2))
    with pytest.raises(Exception, match="4 or 8 waves"):
        ka.gemm_medium(a[:20], packed, 32, "f32", plan=(1, 16, 1))


@pytest.mark.parametrize("width", [120, 203, 3584, 5000])
def test_consumers_add_partial_sums_in_order(width):
    rng = np.random.default_rng(3)
    k = kernels()
    h_ref = rng.normal(size=(5, width)).astype(np.float32)
    parts = rng.normal(size=(4, 5, width)).astype(np.float32)
    weight = np.ones(width, dtype=np.float32)
    h = torch.from_numpy(h_ref.copy()).to(DEVICE)
    out = k.rms_norm(h, torch.from_numpy(weight).to(DEVICE), 1e-5, torch.float32, delta=torch.from_numpy(parts).to(DEVICE), write_h=True)
    total = h_ref.astype(np.float64) + parts.astype(np.float64).sum(axis=0)
    np.testing.assert_allclose(h.cpu().numpy(), total, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(out.cpu().numpy(), plain.rms_norm(total, weight, 1e-5), rtol=1e-5, atol=1e-5)
    picked = torch.tensor([3, 1], dtype=torch.int32, device=DEVICE)      # chosen rows, the stream left as it is
    h = torch.from_numpy(h_ref.copy()).to(DEVICE)
    some = k.rms_norm(h, torch.from_numpy(weight).to(DEVICE), 1e-5, torch.float32, delta=torch.from_numpy(parts).to(DEVICE), rows=picked)
    np.testing.assert_allclose(some.cpu().numpy(), plain.rms_norm(total[[3, 1]], weight, 1e-5), rtol=1e-5, atol=1e-5)
    assert torch.equal(h.cpu(), torch.from_numpy(h_ref))
    heads, kv_heads, hd = 3, 1, 16
    qkv_parts = rng.normal(size=(3, 6, (heads + 2 * kv_heads) * hd)).astype(np.float32)
    positions = torch.arange(6, dtype=torch.int32, device=DEVICE)
    q_parts = k.qkv_rope_store(torch.from_numpy(qkv_parts).to(DEVICE), None, positions, None, None, None, None,
                               heads, kv_heads, hd, 16, torch.float32)
    q_sum = k.qkv_rope_store(torch.from_numpy(qkv_parts.sum(axis=0)).to(DEVICE), None, positions, None, None, None, None,
                             heads, kv_heads, hd, 16, torch.float32)
    np.testing.assert_allclose(q_parts.cpu().numpy(), q_sum.cpu().numpy(), rtol=1e-6, atol=1e-6)


# ---- long contexts ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("window", [0, 5000])
def test_attention_kernels_at_twenty_thousand_keys(window):
    """Block tables hundreds of pages wide, positions beyond 2^14, many splits: all three kernels agree with the plain rule."""
    heads, kv_heads, hd, page_size = 4, 2, 64, 16
    rng = np.random.default_rng(99)
    lengths, counts = [20011, 777, 12000], [150, 1, 40]
    t, q_exact, ek, ev, seq, pos = build_paged_case(rng, torch.bfloat16, lengths, counts, heads, kv_heads, hd, page_size)
    scale = 1.0 / math.sqrt(hd)
    reference = reference_attention(q_exact, ek, ev, seq, pos, heads, kv_heads, hd, scale, window)
    k = kernels()
    tiles = k.pair_query_tiles(query_tile_list(lengths, counts), adjacent=window > 0)
    prefill = k.paged_attention_prefill(t["q"], t["k"], t["v"], t["table"], torch.tensor(tiles, dtype=torch.int32, device=DEVICE),
                                        t["pos"], scale, window, heads, kv_heads, hd)
    np.testing.assert_allclose(prefill.float().cpu().numpy(), reference, **tolerance(torch.bfloat16))
    for splits in (1, 16, 200):
        decode = k.paged_attention_decode(t["q"], t["k"], t["v"], t["table"], t["seq"], t["pos"], scale, window,
                                          heads, kv_heads, hd, splits)
        np.testing.assert_allclose(decode.float().cpu().numpy(), reference, **tolerance(torch.bfloat16))
    rowwise = k.paged_attention_rowwise(t["q"], t["k"], t["v"], t["table"], t["seq"], t["pos"], scale, window, heads, kv_heads, hd)
    np.testing.assert_allclose(rowwise.float().cpu().numpy(), reference, **tolerance(torch.bfloat16))


def test_measured_peaks_are_plausible():
    peaks = kernels().measured_peaks(read_bytes=1 << 30)
    assert 2000.0 < peaks["hbm_read_GBps"] <= 8000.0, "a read-only kernel reaches between a quarter of and the published HBM peak"
    assert 500.0 < peaks["mfma_bf16_TFLOPs"] <= 2500.0, "an MFMA-only kernel reaches at most the published dense bfloat16 peak"


def test_library_tuning_keeps_the_product_and_is_switched_per_shape(tmp_path):
    """With tuning on, a large bfloat16 product is tuned once per shape (PyTorch's TunableOp) and still the product;
    small ones and float32 results go the usual way."""
    import torch.cuda.tunable as tunable
    ka = kernels()
    rng = np.random.default_rng(3)
    a_ref, a = to_bf16_exact(rng.normal(size=(ka.LIBRARY_TUNE_ROWS, 64)))
    w_ref, w = to_bf16_exact(rng.normal(size=(48, 64)) * 0.1)
    expected = a_ref @ w_ref.T
    before = ka.gemm_bf16(a, w)
    ka.set_library_tuning(True, results_file=str(tmp_path / "results.csv"))
    try:
        assert ka.library_tuning() and tunable.is_enabled() and not tunable.tuning_is_enabled()
        tuned = ka.gemm_bf16(a, w)
        assert (ka.LIBRARY_TUNE_ROWS, 48, 64) in ka._library_tuning["seen"] and not tunable.tuning_is_enabled()
        again = ka.gemm_bf16(a, w)
        assert torch.equal(tuned, again)
        for out in (before, tuned):
            assert np.abs(out.float().cpu().numpy() - expected).max() <= 5e-3 * np.abs(expected).max()
        small = ka.gemm_bf16(a[:100].contiguous(), w)
        assert (100, 48, 64) not in ka._library_tuning["seen"]
        assert np.abs(small.float().cpu().numpy() - expected[:100]).max() <= 5e-3 * np.abs(expected).max()
        wide = ka.gemm_bf16(a, w, torch.float32)
        assert np.abs(wide.double().cpu().numpy() - expected).max() <= 1e-5 * np.abs(expected).max()
    finally:
        ka.set_library_tuning(False)
    assert not ka.library_tuning() and not tunable.is_enabled()


# ---- the products at the largest sizes the engine runs: a full vocabulary, the widths of the largest model ---------
def float32_oracle(a, w):
    """``a @ w.T`` of the widened bfloat16 operands, in true float32 on the GPU with a long double check on a sample:
    an oracle that does not share a line with the kernels and fits the memory at these sizes."""
    previous = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        expected = a.float() @ w.float().t()
    finally:
        torch.backends.cuda.matmul.allow_tf32 = previous
    rng = np.random.default_rng(0)
    rows, cols = rng.integers(0, a.shape[0], size=64), rng.integers(0, w.shape[0], size=64)
    exact = (a[rows].double() * w[cols].double()).sum(dim=1)
    scale = expected.abs().max().item()
    assert (expected[rows, cols].double() - exact).abs().max().item() <= 2e-6 * scale
    return expected


@pytest.mark.parametrize("n,k", [(152064, 3584), (152064, 8192), (8192, 29568), (2 * 29568, 8192)])
def test_products_at_full_vocabulary_and_the_largest_widths(n, k):
    """The head over 152 064 tokens and the projections of hidden 8192 / intermediate 29 568, through each of the
    three products, against a float32 product of the same operands: skinny at 1, 8 and 16 rows, medium at 17 and
    64, tiled at 300 (two tiles of rows, the second ragged)."""
    ka = kernels()
    generator = torch.Generator(device=DEVICE).manual_seed(n + k)
    w = (torch.randn((n, k), generator=generator, device=DEVICE) * 0.05).to(torch.bfloat16)
    a = torch.randn((300, k), generator=generator, device=DEVICE).to(torch.bfloat16)
    a[7, 100] = 50.0          # one large entry: a row whose sum a wrong k range or a dropped tail would miss
    w[n - 1, k - 1] = 1.0     # the last element of the last row counts
    a[0, k - 1] = 30.0
    packed = ka.pack_weight(w)
    expected = float32_oracle(a, w)
    scale = expected.abs().max().item()

    def check(out, rows, bound):
        assert out.shape == (rows, n)
        error = (out.float() - expected[:rows]).abs().max().item()
        assert error <= bound * scale, f"n {n} k {k} rows {rows}: error {error / scale:.2e} of the scale"

    if n == 152064:           # the float32 path's product (one thread per output, ascending k) over the same operands
        wide = w.float()
        check(ka.gemm_f32(a[:5].float().contiguous(), wide), 5, 2e-5)
        del wide
    for rows in (1, 8, 16):
        check(ka.gemm_skinny(a[:rows].contiguous(), packed, n, "f32"), rows, 2e-5)
    check(ka.gemm_skinny(a[:16].contiguous(), packed, n, "bf16"), 16, 5e-3)
    for rows in (17, 64):
        out = ka.gemm_medium(a[:rows].contiguous(), packed, n, "f32")
        check(out.sum(dim=0) if out.dim() == 3 else out, rows, 2e-5)
        check(ka.gemm_medium(a[:rows].contiguous(), packed, n, "bf16"), rows, 5e-3)
    check(ka.gemm_tiled(a, packed, n, "f32"), 300, 2e-5)
    check(ka.gemm_tiled(a, packed, n, "bf16"), 300, 5e-3)
    splits = ka.tiled_splits(300, n, k)
    if splits > 1:
        check(ka.gemm_tiled(a, packed, n, "f32", splits=splits).sum(dim=0), 300, 2e-5)
    if n == 2 * 29568:        # gate and up of the largest feed-forward: the gated epilogues
        gated = ka.pack_weight(w, interleave_halves=True)
        want = torch.nn.functional.silu(expected[:, :n // 2]) * expected[:, n // 2:]
        bound = 1.2e-2 * want.abs().max().item()
        for rows, product in ((16, ka.gemm_skinny), (40, ka.gemm_medium), (300, ka.gemm_tiled)):
            got = product(a[:rows].contiguous(), gated, n, "gated")
            assert got.shape == (rows, n // 2) and (got.float() - want[:rows]).abs().max().item() <= bound
