"""Each HIP kernel alone against the plain NumPy function of the same formula, at sizes the tiny
models do not use.  Held vectors of the reference's own kernel tests are restated where they exist
(tests/test_kernels.cu, tests/test_paged_attention.cu)."""
import math

import numpy as np
import pytest
import torch

import plain_llama as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from kvcm_amd import ops as _ops
    _ops.lib()
    return _ops


def _t(a, dtype):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def _np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def _vt(vc, dtype):
    """A value cache built as [pages, kv_heads, slot, dim] in the layout the kernels read:
    [pages, kv_heads, dim, slot]."""
    return torch.tensor(np.ascontiguousarray(np.asarray(vc).transpose(0, 1, 3, 2)), dtype=dtype, device=DEV)


def _bf16_grid(a):
    return plain.round_bf16(a)


# ------------------------------------------------------------------------------- embedding
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_gathers_rows(ops, dtype):
    rng = np.random.default_rng(0)
    V, H = 387, 100
    table = _bf16_grid(rng.normal(size=(V, H)))
    ids = np.array([0, 386, 5, 5, 17], dtype=np.int32)
    out = torch.zeros(len(ids), H, dtype=torch.float32, device=DEV)
    ops.embed(_t(ids, torch.int32), _t(table, dtype), out)
    np.testing.assert_array_equal(_np(out), plain.embedding(table, ids))


# -------------------------------------------------------------------------------- RMS norm
def test_rmsnorm_with_row_gather_reference_vector(ops):
    # tests/test_kernels.cu:25-49: R=5, H=2048, rows {4,0,2}, x ~ 3 N(0,1), w ~ 1 + 0.1 N, eps 1e-5
    rng = np.random.default_rng(1)
    R, H = 5, 2048
    x = (rng.normal(size=(R, H)) * 3).astype(np.float32)
    w = _bf16_grid(1 + 0.1 * rng.normal(size=H))
    rows = np.array([4, 0, 2], dtype=np.int32)
    out = torch.zeros(3, H, dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(_t(x, torch.float32), _t(w, torch.bfloat16), out, 1e-5, rows=_t(rows, torch.int32))
    ref = plain.rms_norm(x[rows], w, 1e-5, plain.round_bf16)
    got = _np(out)
    # one bfloat16 step at most (a product that lands on a rounding tie in one of the two)
    assert np.max(np.abs(got - ref) / np.maximum(1.0, np.abs(ref))) <= 2 ** -7
    assert np.mean(got == ref) > 0.995
    out32 = torch.zeros(3, H, dtype=torch.float32, device=DEV)
    ops.rmsnorm(_t(x, torch.float32), _t(w, torch.float32), out32, 1e-5, rows=_t(rows, torch.int32))
    np.testing.assert_allclose(_np(out32), plain.rms_norm(x[rows], w, 1e-5), rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("H", [96, 1000, 4099])
def test_rmsnorm_fused_add_updates_the_stream(ops, H):
    rng = np.random.default_rng(2)
    T = 7
    x = rng.normal(size=(T, H)).astype(np.float32)
    y = rng.normal(size=(T, H)).astype(np.float32)
    w = rng.normal(size=H).astype(np.float32)
    xt = _t(x, torch.float32)
    out = torch.zeros(T, H, dtype=torch.float32, device=DEV)
    ops.rmsnorm(xt, _t(w, torch.float32), out, 1e-6, add=_t(y, torch.float32))
    np.testing.assert_array_equal(_np(xt), (x + y).astype(np.float64))
    np.testing.assert_allclose(_np(out), plain.rms_norm((x + y).astype(np.float64), w, 1e-6), rtol=3e-6, atol=1e-6)
    # gathered add: the stream is left alone
    xt = _t(x, torch.float32)
    rows = _t([6, 1], torch.int32)
    out = torch.zeros(2, H, dtype=torch.float32, device=DEV)
    ops.rmsnorm(xt, _t(w, torch.float32), out, 1e-6, add=_t(y, torch.float32), rows=rows)
    np.testing.assert_array_equal(_np(xt), x.astype(np.float64))
    np.testing.assert_allclose(_np(out), plain.rms_norm((x + y)[[6, 1]].astype(np.float64), w, 1e-6), rtol=3e-6, atol=1e-6)


def test_rmsnorm_eps_is_inside_the_root(ops):
    # x = c * ones, w = 1  ->  c / sqrt(c^2 + eps); with eps as large as c^2 a misplaced eps shows
    H, c, eps = 64, 0.01, 1e-4
    out = torch.zeros(1, H, dtype=torch.float32, device=DEV)
    ops.rmsnorm(torch.full((1, H), c, device=DEV), torch.ones(H, device=DEV), out, eps)
    np.testing.assert_allclose(_np(out), c / math.sqrt(c * c + eps), rtol=1e-6)


# ---------------------------------------------------------------------------------- rotary
def _inv_freq(hd, theta):
    j = np.arange(hd // 2, dtype=np.float32)
    return (np.float32(1.0) / np.power(np.float32(theta), (np.float32(2.0) * j) / np.float32(hd))).astype(np.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_matches_rotate_half_reference_vector(ops, dtype):
    # tests/test_kernels.cu:51-78: T=3, NH=4, NKV=2, HD=64, positions {0,7,1999}, theta 1e4
    rng = np.random.default_rng(3)
    T, NH, NKV, HD = 3, 4, 2, 64
    qkv = _bf16_grid(rng.normal(size=(T, (NH + 2 * NKV) * HD)))
    pos = np.array([0, 7, 1999], dtype=np.int32)
    t = _t(qkv, dtype)
    ops.rope_cache(t, NH, NKV, HD, positions=_t(pos, torch.int32), inv_freq=_t(_inv_freq(HD, 1e4), torch.float32))
    got = _np(t).reshape(T, NH + 2 * NKV, HD)
    src = qkv.reshape(T, NH + 2 * NKV, HD)
    r16 = plain.round_bf16 if dtype == torch.bfloat16 else None
    ref = plain.rotary(src[:, :NH + NKV], pos, 1e4, r16)
    tol = 2 ** -5 if dtype == torch.bfloat16 else 1e-5     # |values| < 8: one bfloat16 step there
    np.testing.assert_allclose(got[:, :NH + NKV], ref, atol=tol, rtol=0)
    np.testing.assert_array_equal(got[:, NH + NKV:], src[:, NH + NKV:])        # v heads untouched
    np.testing.assert_array_equal(got[0], src[0])                               # position 0 is the identity
    # each (j, j + hd/2) pair keeps its length
    n0 = src[:, :NH + NKV, :HD // 2] ** 2 + src[:, :NH + NKV, HD // 2:] ** 2
    n1 = got[:, :NH + NKV, :HD // 2] ** 2 + got[:, :NH + NKV, HD // 2:] ** 2
    np.testing.assert_allclose(n1, n0, rtol=3e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-3 if dtype == torch.bfloat16 else 1e-6)


def test_rope_dot_products_depend_on_distance_only(ops):
    rng = np.random.default_rng(4)
    HD = 48
    q = rng.normal(size=(1, HD)).astype(np.float32)
    k = rng.normal(size=(1, HD)).astype(np.float32)
    inv = _t(_inv_freq(HD, 5e5), torch.float32)

    def dot(pq, pk):
        row = _t(np.concatenate([q, k, k], axis=1), torch.float32)   # one q head, one k head, one v head
        rows = torch.cat([row, row])
        ops.rope_cache(rows, 1, 1, HD, positions=_t([pq, pk], torch.int32), inv_freq=inv)
        a = _np(rows)
        return float(a[0, :HD] @ a[1, HD:2 * HD])

    base = dot(5, 2)
    assert abs(dot(105, 102) - base) < 1e-4 and abs(dot(17, 14) - base) < 1e-4
    assert abs(dot(5, 3) - base) > 1e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_from_a_step_table_equals_rope_with_inline_angles(ops, dtype):
    rng = np.random.default_rng(41)
    T, NH, NKV, HD = 7, 3, 1, 80
    qkv = _bf16_grid(rng.normal(size=(T, (NH + 2 * NKV) * HD)))
    pos = _t(np.array([0, 1, 63, 64, 1000, 4095, 100000], dtype=np.int32), torch.int32)
    inv = _t(_inv_freq(HD, 5e5), torch.float32)
    a, b = _t(qkv, dtype), _t(qkv, dtype)
    table = torch.empty(T, HD // 2, 2, device=DEV)
    ops.rope_table(pos, inv, table)
    ops.rope_cache(a, NH, NKV, HD, positions=pos, inv_freq=inv)
    ops.rope_cache(b, NH, NKV, HD, positions=pos, inv_freq=inv, cos_sin=table)
    assert torch.equal(a, b)
    ang = _np(pos)[:, None].astype(np.float32) * _np(inv)[None, :].astype(np.float32)
    np.testing.assert_allclose(_np(table)[..., 0], np.cos(ang.astype(np.float64)), atol=2e-6)
    np.testing.assert_allclose(_np(table)[..., 1], np.sin(ang.astype(np.float64)), atol=2e-6)


# ------------------------------------------------------------------------------- KV write
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_reshape_and_cache_scatters_to_slots(ops, dtype):
    # tests/test_paged_attention.cu:230-265: T=37, KVH=4, HD=64, B=16, NB=10, padded stride,
    # random slot permutation, slot -1 skipped and its natural slot stays zero
    rng = np.random.default_rng(5)
    T, KVH, HD, B, NB, NH = 37, 4, 64, 16, 10, 4
    stride = (NH + 2 * KVH) * HD + 24
    rows = _bf16_grid(rng.normal(size=(T, stride)))
    slots = rng.permutation(NB * B)[:T].astype(np.int32)
    skipped = 11
    natural = slots[skipped]
    slots[skipped] = -1
    kc = torch.zeros(NB, KVH, B, HD, dtype=dtype, device=DEV)
    vc = torch.zeros(NB, KVH, HD, B, dtype=dtype, device=DEV)        # values lie transposed inside a page
    buf = _t(rows, dtype)
    ops.rope_cache(buf[:, :stride], NH, KVH, HD, slots=_t(slots, torch.int32), kcache=kc, vcache=vc, block_size=B)
    K, V = _np(kc), _np(vc).transpose(0, 1, 3, 2)
    for t in range(T):
        k_src = rows[t, NH * HD:(NH + KVH) * HD].reshape(KVH, HD)
        v_src = rows[t, (NH + KVH) * HD:(NH + 2 * KVH) * HD].reshape(KVH, HD)
        if slots[t] < 0:
            assert not K[natural // B, :, natural % B].any() and not V[natural // B, :, natural % B].any()
            continue
        np.testing.assert_array_equal(K[slots[t] // B, :, slots[t] % B], k_src)
        np.testing.assert_array_equal(V[slots[t] // B, :, slots[t] % B], v_src)
    assert np.count_nonzero(K.any(axis=(1, 3))) == T - 1            # nothing else was touched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,first_slots", [(16, [0]), (16, [37]), (8, [5, 64]), (32, [100, 3]), (16, [7, 72, 16 * 9 + 15])])
def test_values_of_runs_of_consecutive_slots_reach_their_transposed_pages(ops, dtype, B, first_slots):
    """Rows whose slots are consecutive (a prompt portion) are stored to the value pages eight at a
    time: portions that start at a multiple of eight and elsewhere, several portions in one call (the
    second is then out of step with the first), a row in the middle that is not stored, and rows
    that cross pages.  Every other slot of the cache stays zero."""
    rng = np.random.default_rng(61)
    NH, KVH, HD, NB = 3, 2, 32, 24
    lengths = [45, 23, 9][:len(first_slots)]
    slots = np.concatenate([np.arange(f, f + n) for f, n in zip(first_slots, lengths)]).astype(np.int32)
    assert slots.max() < NB * B and len(set(slots.tolist())) == len(slots)
    T = len(slots)
    skipped = 19
    natural = slots[skipped]
    slots[skipped] = -1
    rows = _bf16_grid(rng.normal(size=(T, (NH + 2 * KVH) * HD)))
    kc = torch.zeros(NB, KVH, B, HD, dtype=dtype, device=DEV)
    vc = torch.zeros(NB, KVH, HD, B, dtype=dtype, device=DEV)
    ops.rope_cache(_t(rows, dtype), NH, KVH, HD, slots=_t(slots, torch.int32), kcache=kc, vcache=vc, block_size=B)
    K, V = _np(kc), _np(vc).transpose(0, 1, 3, 2)
    want_k, want_v = np.zeros_like(K), np.zeros_like(V)
    for t in range(T):
        if slots[t] >= 0:
            want_k[slots[t] // B, :, slots[t] % B] = rows[t, NH * HD:(NH + KVH) * HD].reshape(KVH, HD)
            want_v[slots[t] // B, :, slots[t] % B] = rows[t, (NH + KVH) * HD:].reshape(KVH, HD)
    np.testing.assert_array_equal(K, want_k)
    np.testing.assert_array_equal(V, want_v)
    assert not V[natural // B, :, natural % B].any()


def test_fused_rope_and_cache_write_stores_rotated_keys(ops):
    rng = np.random.default_rng(6)
    T, NH, KVH, HD, B = 5, 6, 2, 32, 8
    rows = rng.normal(size=(T, (NH + 2 * KVH) * HD)).astype(np.float32)
    pos = np.array([3, 4, 5, 40, 41], dtype=np.int32)
    slots = np.array([8, 9, 10, 0, 1], dtype=np.int32)
    kc = torch.zeros(3, KVH, B, HD, device=DEV)
    vc = torch.zeros(3, KVH, HD, B, device=DEV)
    buf = _t(rows, torch.float32)
    ops.rope_cache(buf, NH, KVH, HD, positions=_t(pos, torch.int32), inv_freq=_t(_inv_freq(HD, 1e4), torch.float32),
                   slots=_t(slots, torch.int32), kcache=kc, vcache=vc, block_size=B)
    k_ref = plain.rotary(rows[:, NH * HD:(NH + KVH) * HD].reshape(T, KVH, HD), pos, 1e4)
    K, V = _np(kc), _np(vc).transpose(0, 1, 3, 2)
    for t in range(T):
        np.testing.assert_allclose(K[slots[t] // B, :, slots[t] % B], k_ref[t], atol=1e-5)
        np.testing.assert_array_equal(V[slots[t] // B, :, slots[t] % B],
                                      rows[t, (NH + KVH) * HD:].reshape(KVH, HD).astype(np.float64))


# ---------------------------------------------------------------------------------- SwiGLU
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu(ops, dtype):
    # tests/test_kernels.cu:80-94: T=2, I=300
    rng = np.random.default_rng(7)
    T, I = 2, 300
    gu = _bf16_grid(rng.normal(size=(T, 2 * I)))
    gu[0, :3] = [0.0, 30.0, -30.0]          # silu(0) = 0, silu(x) -> x, silu(-x) -> 0
    out = torch.zeros(T, I, dtype=dtype, device=DEV)
    ops.swiglu(_t(gu, dtype), out)
    r16 = plain.round_bf16 if dtype == torch.bfloat16 else None
    ref = plain.swiglu(gu, r16)
    got = _np(out)
    np.testing.assert_allclose(got, ref, rtol=2 ** -7 if r16 else 2e-6, atol=1e-7)
    assert got[0, 0] == 0.0
    np.testing.assert_allclose(got[0, 1], 30.0 * gu[0, I + 1], rtol=2 ** -7)
    assert abs(got[0, 2]) < 1e-10


# -------------------------------------------------------------------------------- residual
def test_add_residual(ops):
    rng = np.random.default_rng(8)
    x = rng.normal(size=(3, 1001)).astype(np.float32)
    y = _bf16_grid(rng.normal(size=(3, 1001)))
    xt = _t(x, torch.float32)
    ops.add_residual(xt, _t(y, torch.bfloat16))
    np.testing.assert_array_equal(_np(xt), (x + y.astype(np.float32)).astype(np.float64))


# ------------------------------------------------------------------------------------ GEMM
@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (3, 130, 96), (70, 176, 64), (129, 65, 1000), (16, 64, 16), (33, 300, 177)])
def test_gemm_f32_equals_x_wT(ops, M, N, K):
    rng = np.random.default_rng(M * 1000 + N)
    x = rng.normal(size=(M, K)).astype(np.float32)
    w = rng.normal(size=(N, K)).astype(np.float32)
    out = torch.zeros(M, N, device=DEV)
    ops.gemm(_t(x, torch.float32), _t(w, torch.float32), out)
    ref = plain.linear(x, w)
    np.testing.assert_allclose(_np(out), ref, rtol=0, atol=2e-6 * math.sqrt(K) * 4)


def test_gemm_f32_rows_do_not_depend_on_the_batch(ops):
    rng = np.random.default_rng(9)
    K, N = 333, 200
    x = rng.normal(size=(150, K)).astype(np.float32)
    w = _t(rng.normal(size=(N, K)).astype(np.float32), torch.float32)
    full = torch.zeros(150, N, device=DEV)
    ops.gemm(_t(x, torch.float32), w, full)
    for lo, hi in [(0, 1), (17, 19), (60, 100), (149, 150)]:
        part = torch.zeros(hi - lo, N, device=DEV)
        ops.gemm(_t(x[lo:hi], torch.float32), w, part)
        assert torch.equal(part, full[lo:hi]), "a row's sum changed with the rows beside it"


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(1, 16, 32), (5, 100, 96), (64, 64, 64), (70, 176, 200), (200, 333, 1024), (3, 50, 20)])
def test_gemm_bf16_equals_x_wT(ops, M, N, K, out_dtype):
    rng = np.random.default_rng(M * 1000 + N)
    x = _bf16_grid(rng.normal(size=(M, K)))
    w = _bf16_grid(rng.normal(size=(N, K)))
    out = torch.zeros(M, N, dtype=out_dtype, device=DEV)
    ops.gemm(_t(x, torch.bfloat16), _t(w, torch.bfloat16), out)
    ref = plain.linear(x, w)
    if out_dtype == torch.bfloat16:
        np.testing.assert_allclose(_np(out), ref, rtol=2 ** -7, atol=1e-4 * math.sqrt(K))
    else:
        np.testing.assert_allclose(_np(out), ref, rtol=0, atol=3e-6 * math.sqrt(K) * 4)


def test_gemm_bf16_fused_projection_equals_separate_ones(ops):
    # the fused QKV product is the three products stacked
    rng = np.random.default_rng(10)
    x = _t(_bf16_grid(rng.normal(size=(9, 96))), torch.bfloat16)
    ws = [_bf16_grid(rng.normal(size=(n, 96))) for n in (96, 32, 32)]
    fused = torch.zeros(9, 160, dtype=torch.float32, device=DEV)
    ops.gemm(x, _t(np.concatenate(ws), torch.bfloat16), fused)
    col = 0
    for w in ws:
        part = torch.zeros(9, w.shape[0], dtype=torch.float32, device=DEV)
        ops.gemm(x, _t(w, torch.bfloat16), part)
        np.testing.assert_allclose(_np(fused[:, col:col + w.shape[0]]), _np(part), atol=1e-5)
        col += w.shape[0]


# ------------------------------------------------------------------------------- attention
def _paged_problem(rng, ctx_lens, nh, nkv, hd, B, all_rows, shuffle=True, spare=7, dtype=torch.float32):
    """Random Q/K/V on the bfloat16 grid, block tables over shuffled pages with unused spares
    (tests/test_paged_attention.cu:41,53-64)."""
    S = len(ctx_lens)
    max_blocks = max((c + B - 1) // B for c in ctx_lens)
    total = sum((c + B - 1) // B for c in ctx_lens)
    nb = total + spare
    phys = np.arange(nb)
    if shuffle:
        np.random.default_rng(77).shuffle(phys)
    Kl = [_bf16_grid(rng.normal(size=(c, nkv, hd))) for c in ctx_lens]
    Vl = [_bf16_grid(rng.normal(size=(c, nkv, hd))) for c in ctx_lens]
    tables = np.zeros((S, max_blocks), dtype=np.int32)
    Kc = np.zeros((nb, nkv, B, hd))
    Vc = np.zeros((nb, nkv, B, hd))
    nxt = 0
    for s, c in enumerate(ctx_lens):
        for b in range((c + B - 1) // B):
            tables[s, b] = phys[nxt]
            nxt += 1
        for t in range(c):
            Kc[tables[s, t // B], :, t % B] = Kl[s][t]
            Vc[tables[s, t // B], :, t % B] = Vl[s][t]
    row_seq, ctx = [], []
    for s, c in enumerate(ctx_lens):
        if all_rows:
            row_seq += [s] * c
            ctx += list(range(1, c + 1))
        else:
            row_seq.append(s)
            ctx.append(c)
    R = len(row_seq)
    Q = _bf16_grid(rng.normal(size=(R, nh, hd)))
    return dict(Q=Q, Kl=Kl, Vl=Vl, Kc=Kc, Vc=Vc, tables=tables, row_seq=np.array(row_seq, np.int32),
                ctx=np.array(ctx, np.int32), S=S, R=R, max_blocks=max_blocks)


def _run_attention(ops, P, nh, nkv, hd, dtype, window=0, scale=None):
    out = torch.zeros(P["R"], nh * hd, dtype=dtype, device=DEV)
    ops.attention(_t(P["Q"].reshape(P["R"], nh * hd), dtype), out, _t(P["Kc"], dtype), _vt(P["Vc"], dtype),
                  _t(P["tables"], torch.int32), P["max_blocks"], _t(P["row_seq"], torch.int32), _t(P["ctx"], torch.int32),
                  nh, nkv, hd, scale if scale is not None else 1.0 / math.sqrt(hd), window)
    return _np(out).reshape(P["R"], nh, hd)


def _ref_attention(P, nh, nkv, hd, window=0, scale=None, r16=None):
    ref = np.zeros((P["R"], nh, hd))
    sc = scale if scale is not None else 1.0 / math.sqrt(hd)
    for r in range(P["R"]):
        s, c = P["row_seq"][r], P["ctx"][r]
        ref[r] = plain.attention(P["Q"][r:r + 1], P["Kl"][s][:c], P["Vl"][s][:c], [c - 1], np.arange(c), sc, window, r16)[0]
    return ref


@pytest.mark.parametrize("B", [8, 16, 32, 64])
@pytest.mark.parametrize("ctx", [1, 15, 16, 17, 2047])
def test_paged_attention_decode_rows(ops, B, ctx):
    # tests/test_paged_attention.cu:160-175: four sequences {ctx, ctx/2, 1, min(ctx+3, 2047)}
    rng = np.random.default_rng(B * 10000 + ctx)
    lens = [ctx, max(1, ctx // 2), 1, min(ctx + 3, 2047)]
    P = _paged_problem(rng, lens, 8, 2, 64, B, all_rows=False)
    got = _run_attention(ops, P, 8, 2, 64, torch.float32)
    np.testing.assert_allclose(got, _ref_attention(P, 8, 2, 64), atol=2e-5, rtol=0)
    got16 = _run_attention(ops, P, 8, 2, 64, torch.bfloat16)
    np.testing.assert_allclose(got16, _ref_attention(P, 8, 2, 64), atol=1e-2, rtol=0)   # the reference's bound


@pytest.mark.parametrize("nh,nkv,hd", [(8, 8, 64), (16, 4, 128), (32, 4, 128), (3, 1, 32), (4, 2, 16), (6, 3, 48), (2, 1, 256), (5, 5, 80)])
def test_paged_attention_head_shapes_prefill_rows_causal(ops, nh, nkv, hd):
    # one row per position (tests/test_paged_attention.cu:177-185), head shapes of l.196-206 and more
    rng = np.random.default_rng(nh * 100 + hd)
    P = _paged_problem(rng, [33, 70, 5], nh, nkv, hd, 16, all_rows=True)
    got = _run_attention(ops, P, nh, nkv, hd, torch.float32)
    np.testing.assert_allclose(got, _ref_attention(P, nh, nkv, hd), atol=2e-5, rtol=0)


def test_paged_attention_refuses_unsupported_head_dim(ops):
    P = _paged_problem(np.random.default_rng(0), [4], 2, 1, 20, 4, all_rows=False)
    with pytest.raises(ops.KernelError, match="head_dim"):
        _run_attention(ops, P, 2, 1, 20, torch.float32)


def test_paged_attention_shuffled_layout_is_bit_identical(ops):
    # tests/test_paged_attention.cu:208-219
    a = _paged_problem(np.random.default_rng(11), [200, 37, 64], 8, 2, 64, 16, all_rows=False, shuffle=True)
    b = _paged_problem(np.random.default_rng(11), [200, 37, 64], 8, 2, 64, 16, all_rows=False, shuffle=False)
    assert not np.array_equal(a["tables"], b["tables"])
    for dt in (torch.float32, torch.bfloat16):
        np.testing.assert_array_equal(_run_attention(ops, a, 8, 2, 64, dt), _run_attention(ops, b, 8, 2, 64, dt))


def test_paged_attention_special_cases(ops):
    rng = np.random.default_rng(12)
    nh, nkv, hd, B = 4, 2, 32, 8
    P = _paged_problem(rng, [1, 40], nh, nkv, hd, B, all_rows=False)
    got = _run_attention(ops, P, nh, nkv, hd, torch.float32)
    # one key: the output is that key's value, for each head's own KV head
    for h in range(nh):
        np.testing.assert_allclose(got[0, h], P["Vl"][0][0, h // 2], atol=1e-6)
    # all keys equal: the output is the mean of the values
    P["Kc"][:] = 0.25
    P["Kl"] = [np.full_like(k, 0.25) for k in P["Kl"]]
    got = _run_attention(ops, P, nh, nkv, hd, torch.float32)
    for h in range(nh):
        np.testing.assert_allclose(got[1, h], P["Vl"][1][:, h // 2].mean(0), atol=1e-6)


def test_paged_attention_equals_dense_library_attention(ops):
    # plain attention without rotation: a library routine with K/V repeated per group
    rng = np.random.default_rng(13)
    nh, nkv, hd, B, n = 6, 2, 64, 16, 50
    P = _paged_problem(rng, [n], nh, nkv, hd, B, all_rows=True)
    got = _run_attention(ops, P, nh, nkv, hd, torch.float32)
    q = torch.tensor(P["Q"]).permute(1, 0, 2)[None]
    k = torch.tensor(P["Kl"][0]).permute(1, 0, 2).repeat_interleave(nh // nkv, 0)[None]
    v = torch.tensor(P["Vl"][0]).permute(1, 0, 2).repeat_interleave(nh // nkv, 0)[None]
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)[0].permute(1, 0, 2).numpy()
    np.testing.assert_allclose(got, ref, atol=2e-5)


def test_paged_attention_finds_a_far_key_among_hundreds(ops):
    # one key far back (and across a page edge) is made to dominate; a lost page or a wrong
    # table row would miss it
    rng = np.random.default_rng(14)
    nh, nkv, hd, B = 4, 1, 64, 16
    for far in (0, 15, 16, 31, 500, 1023):
        P = _paged_problem(rng, [1024], nh, nkv, hd, B, all_rows=False)
        P["Q"][0, 2] = 0.0
        P["Q"][0, 2, 5] = 40.0
        kvec = np.zeros(hd)
        kvec[5] = 40.0
        P["Kl"][0][far, 0] = kvec
        P["Kc"][P["tables"][0, far // B], 0, far % B] = kvec
        got = _run_attention(ops, P, nh, nkv, hd, torch.float32, scale=1.0)
        np.testing.assert_allclose(got[0, 2], P["Vl"][0][far, 0], atol=1e-5)


@pytest.mark.parametrize("window", [1, 5, 16, 17, 64, 100])
def test_paged_attention_window_edge(ops, window):
    rng = np.random.default_rng(15 + window)
    nh, nkv, hd, B = 2, 1, 32, 8
    P = _paged_problem(rng, [130], nh, nkv, hd, B, all_rows=True)
    got = _run_attention(ops, P, nh, nkv, hd, torch.float32, window=window)
    np.testing.assert_allclose(got, _ref_attention(P, nh, nkv, hd, window=window), atol=2e-5)
    # the key just outside the window must be invisible: make it huge for the last row
    r, edge = P["R"] - 1, 130 - 1 - window
    if edge >= 0:
        P["Q"][r, 0] = 0
        P["Q"][r, 0, 3] = 30.0
        kvec = np.zeros(hd)
        kvec[3] = 30.0
        P["Kl"][0][edge, 0] = kvec
        P["Kc"][P["tables"][0, edge // B], 0, edge % B] = kvec
        got = _run_attention(ops, P, nh, nkv, hd, torch.float32, window=window, scale=1.0)
        ref = _ref_attention(P, nh, nkv, hd, window=window, scale=1.0)
        np.testing.assert_allclose(got[r], ref[r], atol=2e-5)
        assert np.abs(got[r, 0] - P["Vl"][0][edge, 0]).max() > 0.1


# -------------------------------------------------------------------------------- sampling
def test_argmax_reference_vector(ops):
    # tests/test_kernels.cu:96-109
    rng = np.random.default_rng(16)
    R, V = 3, 32000
    logits = rng.normal(size=(R, V)).astype(np.float32)
    logits[0, 31999] = 50
    logits[1, 7] = 50
    logits[1, 9] = 50
    logits[2, 12345] = 50
    out = torch.zeros(R, dtype=torch.int32, device=DEV)
    ops.sample(_t(logits, torch.float32), out)
    assert out.tolist() == [31999, 7, 12345]


def test_temperature_sampling_matches_the_plain_draw(ops):
    rng = np.random.default_rng(17)
    R, V = 6, 1000
    logits = rng.normal(size=(R, V)).astype(np.float32)
    temps = np.array([0.0, 0.8, 0.8, 1.5, 0.1, 0.8], dtype=np.float32)
    seeds = np.array([5, 5, 5, 99, 99, 6], dtype=np.int64)
    reqs = np.array([0, 0, 1, 3, 3, 0], dtype=np.int64)
    idx = np.array([0, 0, 0, 7, 8, 0], dtype=np.int32)
    out = torch.zeros(R, dtype=torch.int32, device=DEV)
    ops.sample(_t(logits, torch.float32), out, _t(temps, torch.float32), _t(seeds, torch.int64), _t(reqs, torch.int64),
               _t(idx, torch.int32))
    got = out.tolist()
    for r in range(R):
        want, margin = plain.sample_row(logits[r], float(temps[r]), int(seeds[r]), int(reqs[r]), int(idx[r]))
        assert got[r] == want or (margin is not None and margin < 1e-5)
    assert got[1] != got[2] or got[1] != got[5]          # request id and seed enter the draw


def test_temperature_sampling_follows_softmax(ops):
    logits = np.log(np.array([[0.1, 0.2, 0.3, 0.4]], dtype=np.float64)).astype(np.float32)
    N = 4000
    rows = _t(np.repeat(logits, N, axis=0), torch.float32)
    out = torch.zeros(N, dtype=torch.int32, device=DEV)
    ops.sample(rows, out, torch.full((N,), 1.0, device=DEV), torch.arange(N, device=DEV, dtype=torch.int64),
               torch.zeros(N, dtype=torch.int64, device=DEV), torch.zeros(N, dtype=torch.int32, device=DEV))
    freq = np.bincount(out.cpu().numpy(), minlength=4) / N
    np.testing.assert_allclose(freq, [0.1, 0.2, 0.3, 0.4], atol=0.03)


# ----------------------------------------------------------- decode-shaped product, split K
@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(2048, 2048), (2560, 2048), (11264, 2048), (2048, 5632), (48, 64), (16, 192), (320, 128)])
def test_gemm_skinny_with_and_without_splits(ops, M, N, K):
    rng = np.random.default_rng(M * 7 + N)
    x = _bf16_grid(rng.normal(size=(M, K)))
    w = _bf16_grid(rng.normal(size=(N, K)) * 0.05)
    ref = plain.linear(x, w)
    S = ops.skinny_splits(M, N, K)
    assert S >= 1
    xt, wt = _t(x, torch.bfloat16), _t(w, torch.bfloat16)
    for dtype in (torch.bfloat16, torch.float32):
        out = torch.zeros(M, N, dtype=dtype, device=DEV)
        scratch = torch.zeros(max(S, 1) * M * N, dtype=torch.float32, device=DEV)
        got = ops.gemm(xt, wt, out, scratch=scratch)
        assert got is out
        tol = dict(rtol=2 ** -7, atol=1e-3) if dtype == torch.bfloat16 else dict(rtol=0, atol=2e-5 * math.sqrt(K))
        np.testing.assert_allclose(_np(out), ref, **tol)
        again = torch.zeros_like(out)
        ops.gemm(xt, wt, again, scratch=scratch)
        assert torch.equal(again, out), "the same product gave another result on a second run"
    # without scratch the kernel runs unsplit and still gives the product
    out = torch.zeros(M, N, dtype=torch.float32, device=DEV)
    ops.gemm(xt, wt, out)
    np.testing.assert_allclose(_np(out), ref, rtol=0, atol=2e-5 * math.sqrt(K))


@pytest.mark.parametrize("M", [65, 96, 100, 128, 129, 300, 512])
@pytest.mark.parametrize("N,K", [(2048, 2048), (2560, 512), (192, 320)])
def test_gemm_shared_rows_beyond_64_rows(ops, M, N, K):
    """The weight-streaming kernel for up to 512 rows (row blocks of 128), which the engine uses
    where the library product may not run: inside captured graphs."""
    rng = np.random.default_rng(M + N)
    x = _bf16_grid(rng.normal(size=(M, K)))
    w = _bf16_grid(rng.normal(size=(N, K)) * 0.05)
    ref = plain.linear(x, w)
    xt, wt = _t(x, torch.bfloat16), _t(w, torch.bfloat16)
    keep, ops.LIBRARY_GEMM_MIN_ROWS = ops.LIBRARY_GEMM_MIN_ROWS, 0
    try:
        S = ops.skinny_splits(M, N, K)
        assert S >= 1
        scratch = torch.zeros(S * M * N, dtype=torch.float32, device=DEV)
        out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
        ops.gemm(xt, wt, out, scratch=scratch)
        np.testing.assert_allclose(_np(out), ref, rtol=2 ** -7, atol=1e-3)
        out32 = torch.zeros(M, N, dtype=torch.float32, device=DEV)
        ops.gemm(xt, wt, out32)                                             # unsplit
        np.testing.assert_allclose(_np(out32), ref, rtol=0, atol=2e-5 * math.sqrt(K))
        if N % 64 == 0 and N >= 2048:                                       # gate/up with the SwiGLU epilogue
            I = N // 2
            act = torch.zeros(M, I, dtype=torch.bfloat16, device=DEV)
            if ops.gemm_swiglu(xt, wt, act):
                want = torch.zeros_like(act)
                ops.swiglu(out, want)
                a, b = _np(act), _np(want)
                assert np.mean(a == b) > 0.98
                np.testing.assert_allclose(a, b, rtol=2 ** -6, atol=2e-3)
    finally:
        ops.LIBRARY_GEMM_MIN_ROWS = keep


def test_gemm_shared_rows_with_every_number_of_waves(ops):
    """The shared-rows kernel sizes its workgroups (two to eight waves, one column tile each) so that tiles x
    splits come to about one workgroup per CU: every number of waves, plain and with the SwiGLU epilogue, with a
    last workgroup that has fewer tiles than waves, against the 64-bit product."""
    keep, ops.LIBRARY_GEMM_MIN_ROWS = ops.LIBRARY_GEMM_MIN_ROWS, 0
    seen, seen_act = set(), set()
    try:
        for M, N, K in [(24, 1024, 2048), (32, 2560, 2048), (64, 2560, 2048), (64, 2560, 8192), (40, 6144, 1024),
                        (100, 7168, 1024), (33, 8192, 1024), (96, 2048, 2048)]:
            rng = np.random.default_rng(M + N + K)
            x = _bf16_grid(rng.normal(size=(M, K)))
            w = _bf16_grid(rng.normal(size=(N, K)) * 0.05)
            ref = plain.linear(x, w)
            S = ops.skinny_splits(M, N, K)
            waves = ops.skinny_waves(M, N, K, S)
            assert S > 1 and 2 <= waves <= 8 and (N // 16 + waves - 1) // waves * S <= 256 + 64, (M, N, K, S, waves)
            seen.add(waves)
            scratch = torch.zeros(S * M * N, dtype=torch.float32, device=DEV)
            out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
            ops.gemm(_t(x, torch.bfloat16), _t(w, torch.bfloat16), out, scratch=scratch)
            np.testing.assert_allclose(_np(out), ref, rtol=2 ** -7, atol=1e-3, err_msg=f"{M}x{N}x{K}: {waves} waves, {S} splits")
        for M, I, K in [(32, 5120, 256), (64, 5632, 256), (24, 5632, 256), (48, 10240, 128), (96, 11008, 128),
                        (17, 14336, 128), (128, 14336, 128), (20, 16384, 128)]:
            rng = np.random.default_rng(M + I + K)
            x = _bf16_grid(rng.normal(size=(M, K)))
            w = _bf16_grid(rng.normal(size=(2 * I, K)) * 0.2)
            waves = ops.skinny_waves(M, I, K, 1, swiglu=True)
            assert 2 <= waves <= 8
            seen_act.add(waves)
            xt, wt = _t(x, torch.bfloat16), _t(w, torch.bfloat16)
            act = torch.full((M, I), 7.0, dtype=torch.bfloat16, device=DEV)
            assert ops.gemm_swiglu(xt, wt, act)
            gu = torch.zeros(M, 2 * I, dtype=torch.bfloat16, device=DEV)
            ops.gemm(xt, wt, gu)                                 # unsplit: no scratch given
            want = torch.zeros_like(act)
            ops.swiglu(gu, want)
            a, b = _np(act), _np(want)
            # the two launches walk K from different starting points: a sum may round to the neighbouring bfloat16
            # (2^-7 relative), in the gate, in the up value, or in both, and SiLU below zero multiplies a step of
            # its argument by up to four
            assert np.mean(a == b) > 0.98, f"{M}x{I}x{K}: {waves} waves"
            np.testing.assert_allclose(a, b, rtol=2 ** -5, atol=2e-3, err_msg=f"{M}x{I}x{K}: {waves} waves")
    finally:
        ops.LIBRARY_GEMM_MIN_ROWS = keep
    assert seen == {2, 3, 4, 5, 6, 7, 8} and seen_act >= {3, 4, 5, 6, 7, 8}, (seen, seen_act)


def test_long_k_products_of_wide_models_stay_with_this_packages_kernel_up_to_192_rows(ops):
    """From 96 rows on a bfloat16 product is the vendor library's, except those whose K is at least their width and
    whose weights are 32 MB or more, up to 192 rows: the shared-rows kernel takes them, split, and the result is right."""
    assert ops._library_takes(128, 2048, 5632) and ops._library_takes(96, 6144, 4096)          # 23 MB; wider than K
    assert not ops._library_takes(128, 4096, 4096) and not ops._library_takes(192, 4096, 14336)
    assert ops._library_takes(193, 4096, 4096) and not ops._library_takes(95, 2048, 2048)
    M, N, K = 150, 4096, 4096
    rng = np.random.default_rng(5)
    x = _bf16_grid(rng.normal(size=(M, K)))
    w = _bf16_grid(rng.normal(size=(N, K)) * 0.03)
    S = ops.skinny_splits(M, N, K)
    assert S > 1
    scratch = torch.zeros(S * M * N, dtype=torch.float32, device=DEV)
    out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
    got = ops.gemm(_t(x, torch.bfloat16), _t(w, torch.bfloat16), out, scratch=scratch, keep_partial=True)
    assert isinstance(got, ops.PartialSums) and got.splits == S          # the library leaves no partial sums
    np.testing.assert_allclose(_np(got.materialize()), plain.linear(x, w), rtol=2 ** -7, atol=2e-3)


@pytest.mark.parametrize("mode", ["off", "heuristic", "all"])
@pytest.mark.parametrize("M,N,K", [(96, 192, 320), (200, 2560, 512), (333, 328, 136)])
def test_library_product_with_each_choice_of_algorithm(ops, mode, M, N, K):
    """Many-row products go to the vendor library; which of its algorithms runs is its heuristic's first
    choice, or the fastest of the timed candidates whose result agrees with that one's.  Whatever was
    chosen, the product is x w^T, the choice is made once per shape, and a view with a row stride works."""
    rng = np.random.default_rng(M + N + K)
    x = _bf16_grid(rng.normal(size=(M, K)))
    w_all = _bf16_grid(rng.normal(size=(N, K + 8)) * 0.05)
    w = w_all[:, :K]
    ref = plain.linear(x, w)
    xt = _t(x, torch.bfloat16)
    wt = _t(w_all, torch.bfloat16)[:, :K]                    # rows K + 8 apart
    keep = ops.LIBRARY_TUNING
    ops.LIBRARY_TUNING = mode
    try:
        shape = (M, N, K, K, K + 8, N)
        want = {"off": 0, "heuristic": 1, "all": 2}[mode]
        out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
        before = len(ops.library_tuning_log)
        ops.gemm(xt, wt, out)
        np.testing.assert_allclose(_np(out), ref, rtol=2 ** -7, atol=1e-3)
        assert ops.lib().kvcm_gemm_library_tuned(*shape) >= want
        logged = len(ops.library_tuning_log)
        assert logged - before <= (1 if want else 0)
        if logged > before:
            m, n, k, first_us, kept_us, timed = ops.library_tuning_log[-1]
            assert (m, n, k) == (M, N, K) and timed >= 1 and 0 < kept_us and 0 < first_us
        again = torch.zeros_like(out)
        ops.gemm(xt, wt, again)                               # the shape is tuned: nothing is timed again
        assert len(ops.library_tuning_log) == logged
        assert torch.equal(again, out)
    finally:
        ops.LIBRARY_TUNING = keep


def test_partial_sums_feed_the_fused_norm_and_rope(ops):
    rng = np.random.default_rng(30)
    M, H, K = 5, 2048, 2048
    x_in = _bf16_grid(rng.normal(size=(M, K)))
    w = _bf16_grid(rng.normal(size=(H, K)) * 0.03)
    S = ops.skinny_splits(M, H, K)
    assert S > 1
    scratch = torch.zeros(S * 64 * H, dtype=torch.float32, device=DEV)
    out = torch.zeros(M, H, dtype=torch.bfloat16, device=DEV)
    part = ops.gemm(_t(x_in, torch.bfloat16), _t(w, torch.bfloat16), out, scratch=scratch, keep_partial=True)
    assert isinstance(part, ops.PartialSums) and part.splits == S
    resid = rng.normal(size=(M, H)).astype(np.float32)
    nw = _bf16_grid(1 + 0.1 * rng.normal(size=H))
    # fused: residual += round(product); out = norm(residual)
    xt = _t(resid, torch.float32)
    normed = torch.zeros(M, H, dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(xt, _t(nw, torch.bfloat16), normed, 1e-5, add=part)
    # unfused: materialise the product, then the ordinary fused add
    prod = part.materialize()
    xt2 = _t(resid, torch.float32)
    normed2 = torch.zeros_like(normed)
    ops.rmsnorm(xt2, _t(nw, torch.bfloat16), normed2, 1e-5, add=prod)
    assert torch.equal(xt, xt2) and torch.equal(normed, normed2)
    np.testing.assert_allclose(_np(prod), plain.linear(x_in, w, plain.round_bf16), rtol=2 ** -7, atol=1e-3)
    # gathered rows, nothing written back
    xt3 = _t(resid, torch.float32)
    g = torch.zeros(2, H, dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(xt3, _t(nw, torch.bfloat16), g, 1e-5, add=part, rows=_t([4, 1], torch.int32))
    assert torch.equal(g, normed[[4, 1]]) and torch.equal(xt3, _t(resid, torch.float32))

    # rotary + cache write from partial sums equals the same from the stored rows
    nh, nkv, hd, B = 24, 4, 64, 16                                   # (24 + 8) * 64 = 2048 columns
    pos = _t([0, 5, 17, 100, 101], torch.int32)
    slots = _t([3, 20, 35, 1, 16], torch.int32)
    inv = _t(_inv_freq(hd, 1e4), torch.float32)
    caches = [torch.zeros(3, nkv, B, hd, dtype=torch.bfloat16, device=DEV) if i % 2 == 0 else
              torch.zeros(3, nkv, hd, B, dtype=torch.bfloat16, device=DEV) for i in range(4)]
    rows_a = prod.clone()
    ops.rope_cache(rows_a, nh, nkv, hd, positions=pos, inv_freq=inv, slots=slots, kcache=caches[0], vcache=caches[1], block_size=B)
    rows_b = torch.zeros_like(rows_a)
    ops.rope_cache(rows_b, nh, nkv, hd, positions=pos, inv_freq=inv, slots=slots, kcache=caches[2], vcache=caches[3],
                   block_size=B, source=part)
    assert torch.equal(rows_a[:, :nh * hd], rows_b[:, :nh * hd])       # q
    assert torch.equal(caches[0], caches[2]) and torch.equal(caches[1], caches[3])


def test_skinny_gemm_with_swiglu_epilogue_equals_product_then_swiglu(ops):
    rng = np.random.default_rng(77)
    for M, I, K in ((8, 2560, 256), (1, 5632, 2048), (37, 2568, 192), (64, 5120, 128), (20, 5120, 192), (40, 5152, 64), (33, 10240, 64)):
        x = _t(rng.normal(size=(M, K)), torch.bfloat16)
        w = _t(rng.normal(size=(2 * I, K)) * 0.1, torch.bfloat16)
        act = torch.zeros(M, I, dtype=torch.bfloat16, device=DEV)
        assert ops.gemm_swiglu(x, w, act)
        gu = torch.zeros(M, 2 * I, dtype=torch.bfloat16, device=DEV)
        ops.gemm(x, w, gu)                                   # unsplit: no scratch given
        ref = torch.zeros_like(act)
        ops.swiglu(gu, ref)
        # the two launches walk K in different orders (other kernels, or workgroups that start at different
        # places): a sum may round to the neighbouring bfloat16 now and then
        a, b = _np(act), _np(ref)
        assert np.mean(a == b) > 0.98
        np.testing.assert_allclose(a, b, rtol=2 ** -6, atol=2e-3)
    small = torch.zeros(8, 256, dtype=torch.bfloat16, device=DEV)      # too few columns to fill the chip unsplit
    assert not ops.gemm_swiglu(_t(rng.normal(size=(8, 64)), torch.bfloat16), _t(rng.normal(size=(512, 64)), torch.bfloat16), small)
    big = torch.zeros(65, 2560, dtype=torch.bfloat16, device=DEV)      # too many rows for the streaming kernel
    assert not ops.gemm_swiglu(_t(rng.normal(size=(65, 64)), torch.bfloat16), _t(rng.normal(size=(5120, 64)), torch.bfloat16), big)


# ------------------------------------------------------------ partitioned decode attention
@pytest.mark.parametrize("nh,nkv,hd", [(32, 4, 64), (8, 8, 64), (16, 4, 128), (32, 4, 128), (6, 2, 64), (5, 1, 128), (7, 7, 64)])
@pytest.mark.parametrize("B", [8, 16, 64])
def test_partitioned_decode_attention(ops, nh, nkv, hd, B):
    rng = np.random.default_rng(nh * 31 + hd + B)
    lens = [700, 256, 257, 1, 255, 33]
    P = _paged_problem(rng, lens, nh, nkv, hd, B, all_rows=False)
    ref = _ref_attention(P, nh, nkv, hd)
    R = P["R"]
    for bound in (max(lens), 2048, 2048):               # the launch may be sized for a longer context
        out = torch.full((R, nh * hd), 9.0, dtype=torch.bfloat16, device=DEV)
        scratch = torch.full((ops.attention_decode_scratch(R, nh, hd, bound),), float("nan"), dtype=torch.float32, device=DEV)
        ops.attention_decode(_t(P["Q"].reshape(R, nh * hd), torch.bfloat16), out, _t(P["Kc"], torch.bfloat16),
                             _vt(P["Vc"], torch.bfloat16), _t(P["tables"], torch.int32), P["max_blocks"],
                             _t(P["row_seq"], torch.int32), _t(P["ctx"], torch.int32), nh, nkv, hd, 1.0 / math.sqrt(hd),
                             bound, scratch)
        np.testing.assert_allclose(_np(out).reshape(R, nh, hd), ref, atol=1e-2, rtol=0)
    generic = _run_attention(ops, P, nh, nkv, hd, torch.bfloat16)
    np.testing.assert_allclose(_np(out).reshape(R, nh, hd), generic, atol=2 ** -6, rtol=0)   # v1 vs v2: a rounding apart


@pytest.mark.parametrize("nh,nkv,hd", [(8, 2, 64), (6, 2, 128)])
def test_partitioned_decode_attention_many_partitions(ops, nh, nkv, hd):
    """Twenty partitions and more: the merge takes them in groups; a key in a middle partition that
    outweighs all others must come through alone, and plain rows must match the plain attention."""
    rng = np.random.default_rng(41 + hd)
    B, lens = 16, [5000, 2300, 257]
    P = _paged_problem(rng, lens, nh, nkv, hd, B, all_rows=False)
    far = 2600                                                # partition 10 of 20
    P["Q"][0, 3] = 0.0
    P["Q"][0, 3, 5] = 40.0
    kvec = np.zeros(hd)
    kvec[5] = 40.0
    kvh = 3 // (nh // nkv)
    P["Kl"][0][far, kvh] = kvec
    P["Kc"][P["tables"][0, far // B], kvh, far % B] = kvec
    ref = _ref_attention(P, nh, nkv, hd, scale=1.0 / math.sqrt(hd))
    for bound in (5000, 8192):
        out = torch.full((3, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
        scratch = torch.full((ops.attention_decode_scratch(3, nh, hd, bound),), float("nan"), dtype=torch.float32, device=DEV)
        ops.attention_decode(_t(P["Q"].reshape(3, nh * hd), torch.bfloat16), out, _t(P["Kc"], torch.bfloat16),
                             _vt(P["Vc"], torch.bfloat16), _t(P["tables"], torch.int32), P["max_blocks"],
                             _t(P["row_seq"], torch.int32), _t(P["ctx"], torch.int32), nh, nkv, hd, 1.0 / math.sqrt(hd),
                             bound, scratch)
        got = _np(out).reshape(3, nh, hd)
        np.testing.assert_allclose(got[0, 3], P["Vl"][0][far, kvh], atol=1e-2)
        np.testing.assert_allclose(got, ref, atol=1e-2, rtol=0)


def test_partitioned_decode_attention_padding_rows_and_far_key(ops):
    rng = np.random.default_rng(40)
    nh, nkv, hd, B = 8, 2, 64, 16
    P = _paged_problem(rng, [900, 10], nh, nkv, hd, B, all_rows=False)
    far = 3                                                   # first partition, while the row spans four
    P["Q"][0, 5] = 0.0
    P["Q"][0, 5, 7] = 40.0
    kvec = np.zeros(hd)
    kvec[7] = 40.0
    P["Kl"][0][far, 1] = kvec
    P["Kc"][P["tables"][0, far // B], 1, far % B] = kvec
    ctx = np.array([900, 10, 0], dtype=np.int32)              # a padding row with no context
    q = np.concatenate([P["Q"].reshape(2, nh * hd), np.ones((1, nh * hd))])
    out = torch.full((3, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    scratch = torch.zeros(ops.attention_decode_scratch(3, nh, hd, 1024), dtype=torch.float32, device=DEV)
    ops.attention_decode(_t(q, torch.bfloat16), out, _t(P["Kc"], torch.bfloat16), _vt(P["Vc"], torch.bfloat16),
                         _t(P["tables"], torch.int32), P["max_blocks"], _t([0, 1, 0], torch.int32), _t(ctx, torch.int32),
                         nh, nkv, hd, 1.0, 1024, scratch)
    got = _np(out).reshape(3, nh, hd)
    np.testing.assert_allclose(got[0, 5], P["Vl"][0][far, 1], atol=1e-2)
    assert not got[2].any()
    with pytest.raises(ops.KernelError, match="scratch too small"):
        ops.attention_decode(_t(q, torch.bfloat16), out, _t(P["Kc"], torch.bfloat16), _vt(P["Vc"], torch.bfloat16),
                             _t(P["tables"], torch.int32), P["max_blocks"], _t([0, 1, 0], torch.int32), _t(ctx, torch.int32),
                             nh, nkv, hd, 1.0, 4096, scratch)
    assert not ops.attention_decode_supported(12, 1, 64, torch.bfloat16) and not ops.attention_decode_supported(4, 2, 48, torch.bfloat16)
    assert not ops.attention_decode_supported(32, 4, 64, torch.bfloat16, block_size=4)
    assert not ops.attention_decode_supported(32, 4, 64, torch.float32)


# ------------------------------------------ rotation + page write + attention in one launch
@pytest.mark.parametrize("nh,nkv,hd,B", [(32, 4, 64, 16), (8, 8, 64, 8), (16, 4, 128, 16), (6, 2, 64, 64), (5, 1, 128, 16)])
@pytest.mark.parametrize("source", ["rows", "partial_sums"])
def test_fused_decode_attention_equals_rope_write_attend(ops, nh, nkv, hd, B, source, copies=1):
    rng = np.random.default_rng(nh + hd + B)
    lens = [700, 256, 257, 1, 255, 33, 513, 1024] * copies    # 1..4 chunks, chunk edges, the first token of a sequence
    P = _paged_problem(rng, lens, nh, nkv, hd, B, all_rows=False)
    R, W = P["R"], (nh + 2 * nkv) * hd
    pos = (P["ctx"] - 1).astype(np.int32)
    k_new = _bf16_grid(rng.normal(size=(R, nkv, hd)))
    v_new = _bf16_grid(rng.normal(size=(R, nkv, hd)))
    rows = np.concatenate([P["Q"].reshape(R, -1), k_new.reshape(R, -1), v_new.reshape(R, -1)], axis=1)
    slots = np.array([P["tables"][s, p // B] * B + p % B for s, p in zip(P["row_seq"], pos)], dtype=np.int32)
    inv = _t(_inv_freq(hd, 1e4), torch.float32)
    table = torch.empty(R, hd // 2, 2, device=DEV)
    ops.rope_table(_t(pos, torch.int32), inv, table)
    args = dict(tables=_t(P["tables"], torch.int32), row_seq=_t(P["row_seq"], torch.int32), ctx=_t(P["ctx"], torch.int32))

    # the last token of every sequence is not in the cache yet: both ways have to put it there
    def caches():
        kc, vc = P["Kc"].copy(), P["Vc"].copy()
        for s_, p_ in zip(P["row_seq"], pos):
            kc[P["tables"][s_, p_ // B], :, p_ % B] = 0
            vc[P["tables"][s_, p_ // B], :, p_ % B] = 0
        return _t(kc, torch.bfloat16), _vt(vc, torch.bfloat16)

    # separately: rotation + page write, then the one-pass kernel
    kc1, vc1 = caches()
    q1 = _t(rows, torch.bfloat16)
    ops.rope_cache(q1, nh, nkv, hd, positions=_t(pos, torch.int32), inv_freq=inv, slots=_t(slots, torch.int32),
                   kcache=kc1, vcache=vc1, block_size=B, cos_sin=table)
    want = torch.zeros(R, nh * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention(q1, want, kc1, vc1, args["tables"], P["max_blocks"], args["row_seq"], args["ctx"], nh, nkv, hd, 1.0 / math.sqrt(hd))

    kc2, vc2 = caches()
    if source == "rows":
        proj = _t(rows, torch.bfloat16)
    else:   # three splits whose sum is the row, none of them on the bfloat16 grid
        noise = rng.normal(size=(2, R, W)) * 0.37
        parts = np.stack([noise[0], noise[1], rows - noise[0] - noise[1]]).astype(np.float32)
        parts[2] += (rows - parts.astype(np.float64).sum(0)).astype(np.float32)
        proj = ops.PartialSums(_t(parts, torch.float32), 3, R, W, torch.zeros(R, W, dtype=torch.bfloat16, device=DEV))
        ref_rows = proj.materialize().clone()
        ops.rope_cache(ref_rows, nh, nkv, hd, positions=_t(pos, torch.int32), inv_freq=inv, slots=_t(slots, torch.int32),
                       kcache=kc1, vcache=vc1, block_size=B, cos_sin=table)
        ops.attention(ref_rows, want, kc1, vc1, args["tables"], P["max_blocks"], args["row_seq"], args["ctx"], nh, nkv, hd,
                      1.0 / math.sqrt(hd))
    got = torch.full((R, nh * hd), 5.0, dtype=torch.bfloat16, device=DEV)
    ops.attention_decode_fused(proj, got, kc2, vc2, args["tables"], P["max_blocks"], args["row_seq"], args["ctx"], nh, nkv, hd,
                               1.0 / math.sqrt(hd), cos_sin=table, slots=_t(slots, torch.int32))
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)                      # the same keys and values reached the pages
    np.testing.assert_allclose(_np(got), _np(want), atol=2 ** -6, rtol=0)        # two kernels, a rounding apart


@pytest.mark.parametrize("source", ["rows", "partial_sums"])
def test_fused_decode_attention_of_many_rows(ops, source):
    """From 512 workgroups on (rows x kv heads) a launch at head_dim 64 takes workgroups of four waves
    instead of eight: 64 rows of 8 kv heads, the same contexts as above."""
    test_fused_decode_attention_equals_rope_write_attend(ops, 16, 8, 64, 16, source, copies=8)


@pytest.mark.parametrize("nh,nkv,hd,B", [(8, 2, 64, 16), (6, 2, 128, 32), (32, 4, 64, 16)])
def test_fused_decode_attention_in_parts(ops, nh, nkv, hd, B):
    """Few rows with long contexts: the launch cuts them into parts of whole chunks and a second
    launch merges them.  The part that holds a row's newest token stores it; a padding row and a
    row of one token ride along; one key in a middle part outweighs all others."""
    rng = np.random.default_rng(nh * 7 + hd + B)
    lens = [5000, 2300, 257, 1, 1025]
    P = _paged_problem(rng, lens, nh, nkv, hd, B, all_rows=False)
    R, W = P["R"], (nh + 2 * nkv) * hd
    far, head = 2600, nh - 1
    kvh = head // (nh // nkv)
    pos = (P["ctx"] - 1).astype(np.int32)
    k_new = _bf16_grid(rng.normal(size=(R, nkv, hd)))
    v_new = _bf16_grid(rng.normal(size=(R, nkv, hd)))
    rows = np.concatenate([P["Q"].reshape(R, -1), k_new.reshape(R, -1), v_new.reshape(R, -1)], axis=1)
    rows = np.concatenate([rows, np.ones((1, W))])                              # + a padding row without context
    slots = np.array([P["tables"][s, p // B] * B + p % B for s, p in zip(P["row_seq"], pos)] + [-1], dtype=np.int32)
    row_seq = np.concatenate([P["row_seq"], [0]]).astype(np.int32)
    ctx = np.concatenate([P["ctx"], [0]]).astype(np.int32)
    inv = _t(_inv_freq(hd, 1e4), torch.float32)
    table = torch.empty(R + 1, hd // 2, 2, device=DEV)
    ops.rope_table(_t(np.concatenate([pos, [0]]), torch.int32), inv, table)
    tables = _t(P["tables"], torch.int32)

    def caches():
        return _t(P["Kc"], torch.bfloat16), _vt(P["Vc"], torch.bfloat16)

    kc1, vc1 = caches()
    q1 = _t(rows, torch.bfloat16)
    ops.rope_cache(q1, nh, nkv, hd, positions=_t(np.concatenate([pos, [0]]), torch.int32), inv_freq=inv,
                   slots=_t(slots, torch.int32), kcache=kc1, vcache=vc1, block_size=B, cos_sin=table)
    want = torch.zeros(R + 1, nh * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention(q1, want, kc1, vc1, tables, P["max_blocks"], _t(row_seq, torch.int32), _t(ctx, torch.int32), nh, nkv, hd,
                  1.0 / math.sqrt(hd))
    for bound in (5000, 8192):
        need = ops.attention_decode_fused_scratch(R + 1, nh, nkv, hd, bound)
        # (few workgroups that read more than 256 KB of keys and values each are cut too: 512 tokens at head_dim 128)
        assert need > 0 and ops.attention_decode_fused_scratch(R + 1, nh, nkv, hd, 1024 if hd == 64 else 512) == 0
        assert (ops.attention_decode_fused_scratch(R + 1, nh, nkv, hd, 1024) > 0) == (hd == 128)
        assert ops.attention_decode_fused_scratch(40, nh, nkv, hd, 1024) == 0      # many workgroups: one part each
        kc2, vc2 = caches()
        got = torch.full((R + 1, nh * hd), 5.0, dtype=torch.bfloat16, device=DEV)
        scratch = torch.full((need,), float("nan"), dtype=torch.float32, device=DEV)
        ops.attention_decode_fused(_t(rows, torch.bfloat16), got, kc2, vc2, tables, P["max_blocks"], _t(row_seq, torch.int32),
                                   _t(ctx, torch.int32), nh, nkv, hd, 1.0 / math.sqrt(hd), cos_sin=table,
                                   slots=_t(slots, torch.int32), max_context=bound, scratch=scratch)
        assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)                  # the new tokens reached their pages, once
        np.testing.assert_allclose(_np(got), _np(want), atol=2 ** -6, rtol=0)
        assert not _np(got)[R].any()
    with pytest.raises(ops.KernelError, match="scratch too small"):
        ops.attention_decode_fused(_t(rows, torch.bfloat16), got, kc2, vc2, tables, P["max_blocks"], _t(row_seq, torch.int32),
                                   _t(ctx, torch.int32), nh, nkv, hd, 1.0, max_context=5000, scratch=scratch[:100])
    # an outstanding key in a middle part, no rotation, nothing stored
    P["Q"][0, head] = 0.0
    P["Q"][0, head, 5] = 40.0
    kvec = np.zeros(hd)
    kvec[5] = 40.0
    P["Kc"][P["tables"][0, far // B], kvh, far % B] = kvec
    rows[:R, :nh * hd] = P["Q"].reshape(R, -1)
    kc3, vc3 = caches()
    ops.attention_decode_fused(_t(rows, torch.bfloat16), got, kc3, vc3, tables, P["max_blocks"], _t(row_seq, torch.int32),
                               _t(ctx, torch.int32), nh, nkv, hd, 1.0, max_context=5000)
    np.testing.assert_allclose(_np(got)[0].reshape(nh, hd)[head], P["Vl"][0][far, kvh], atol=1e-2)


def test_fused_decode_attention_against_plain_far_key_padding_and_no_store(ops):
    rng = np.random.default_rng(91)
    nh, nkv, hd, B = 8, 2, 64, 16
    P = _paged_problem(rng, [900, 300], nh, nkv, hd, B, all_rows=False)
    far = 3                                                   # in the first chunk, while the row spans four
    P["Q"][0, 5] = 0.0
    P["Q"][0, 5, 7] = 40.0
    kvec = np.zeros(hd)
    kvec[7] = 40.0
    P["Kl"][0][far, 1] = kvec
    P["Kc"][P["tables"][0, far // B], 1, far % B] = kvec
    ref = _ref_attention(P, nh, nkv, hd, scale=1.0)
    # no rotation, nothing stored: the cache already holds every token, k and v of the rows are ignored
    rows = np.concatenate([P["Q"].reshape(2, -1), rng.normal(size=(2, 2 * nkv * hd))], axis=1)
    rows = np.concatenate([rows, np.ones((1, rows.shape[1]))])                  # + a padding row without context
    ctx = np.array([900, 300, 0], dtype=np.int32)
    kc, vc = _t(P["Kc"], torch.bfloat16), _vt(P["Vc"], torch.bfloat16)
    kc0, vc0 = kc.clone(), vc.clone()
    out = torch.full((3, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention_decode_fused(_t(rows, torch.bfloat16), out, kc, vc, _t(P["tables"], torch.int32), P["max_blocks"],
                               _t([0, 1, 0], torch.int32), _t(ctx, torch.int32), nh, nkv, hd, 1.0)
    got = _np(out).reshape(3, nh, hd)
    np.testing.assert_allclose(got[:2], ref, atol=1e-2, rtol=0)
    np.testing.assert_allclose(got[0, 5], P["Vl"][0][far, 1], atol=1e-2)
    assert not got[2].any() and torch.equal(kc, kc0) and torch.equal(vc, vc0)
    # slot -1 stores nothing either
    ops.attention_decode_fused(_t(rows, torch.bfloat16), out, kc, vc, _t(P["tables"], torch.int32), P["max_blocks"],
                               _t([0, 1, 0], torch.int32), _t(ctx, torch.int32), nh, nkv, hd, 1.0,
                               slots=_t([-1, -1, -1], torch.int32))
    assert torch.equal(kc, kc0) and torch.equal(vc, vc0)
    assert not ops.attention_decode_fused_supported(12, 1, 64, torch.bfloat16) and not ops.attention_decode_fused_supported(4, 2, 48, torch.bfloat16)
    assert not ops.attention_decode_fused_supported(32, 4, 64, torch.float32)


# ------------------------------------------------------------------- tiled prefill attention
def _run_prefill(ops, P, runs, nh, nkv, hd, scale=None):
    """runs: per sequence (first position, number of rows); rows of P are those positions in order."""
    R = P["R"]
    out = torch.full((R, nh * hd), 3.0, dtype=torch.bfloat16, device=DEV)
    run_start = np.concatenate([[0], np.cumsum([n for _, n in runs])]).astype(np.int32)
    ops.attention_prefill(_t(P["Q"].reshape(R, nh * hd), torch.bfloat16), out, _t(P["Kc"], torch.bfloat16),
                          _vt(P["Vc"], torch.bfloat16), _t(P["tables"], torch.int32), P["max_blocks"], _t(run_start, torch.int32),
                          _t([s for s, _ in runs], torch.int32), len(runs), max(n for _, n in runs), nh, nkv, hd,
                          scale if scale is not None else 1.0 / math.sqrt(hd))
    return _np(out).reshape(R, nh, hd)


def _runs_problem(rng, runs, nh, nkv, hd, B):
    """Sequences whose cache holds start+n tokens; query rows are positions start .. start+n-1."""
    P = _paged_problem(rng, [s + n for s, n in runs], nh, nkv, hd, B, all_rows=True)
    keep, row = [], 0
    for s, n in runs:
        keep += list(range(row + s, row + s + n))
        row += s + n
    P["Q"], P["row_seq"], P["ctx"], P["R"] = P["Q"][keep], P["row_seq"][keep], P["ctx"][keep], len(keep)
    return P


@pytest.mark.parametrize("nh,nkv,hd", [(8, 2, 64), (4, 4, 128), (6, 1, 64), (32, 4, 64)])
@pytest.mark.parametrize("B", [8, 16, 64, 128])
def test_prefill_attention_runs_anywhere(ops, nh, nkv, hd, B):
    rng = np.random.default_rng(nh + hd + B)
    runs = [(0, 130), (0, 1), (77, 2), (200, 1), (15, 64), (63, 65), (0, 16), (31, 17)]
    P = _runs_problem(rng, runs, nh, nkv, hd, B)
    got = _run_prefill(ops, P, runs, nh, nkv, hd)
    ref = _ref_attention(P, nh, nkv, hd)
    np.testing.assert_allclose(got, ref, atol=1.5e-2, rtol=0)
    generic = _run_attention(ops, P, nh, nkv, hd, torch.bfloat16)
    np.testing.assert_allclose(got, generic, atol=2e-2, rtol=0)


@pytest.mark.parametrize("nh,nkv,hd,B", [(8, 2, 64, 16), (4, 4, 128, 8), (32, 4, 64, 32)])
def test_prefill_attention_rotates_unrotated_queries_itself(ops, nh, nkv, hd, B):
    """Given the step's table of cos and sin, the tiled kernel rotates q as it reads it: bit for bit what
    it computes from queries that the rotation kernel rotated (the same pairs, the same 32-bit
    multiply-adds, the same rounding to bfloat16; that kernel has its own test against the plain rotation)."""
    rng = np.random.default_rng(nh * hd + B)
    runs = [(0, 130), (77, 2), (15, 64), (63, 65), (300, 1)]
    P = _runs_problem(rng, runs, nh, nkv, hd, B)
    R, half = P["R"], hd // 2
    pos = np.concatenate([np.arange(s, s + n) for s, n in runs]).astype(np.int32)
    inv_freq = (1.0 / (10000.0 ** (np.arange(half, dtype=np.float64) * 2 / hd))).astype(np.float32)
    table = torch.empty(R, half, 2, dtype=torch.float32, device=DEV)
    ops.rope_table(_t(pos, torch.int32), _t(inv_freq, torch.float32), table)
    q_plain = _t(P["Q"].reshape(R, nh * hd), torch.bfloat16)
    q_rot = q_plain.clone()
    ops.rope_cache(q_rot, nh, 0, hd, cos_sin=table)                      # q heads only, no cache
    run_start = _t(np.concatenate([[0], np.cumsum([n for _, n in runs])]).astype(np.int32), torch.int32)
    args = (_t(P["Kc"], torch.bfloat16), _vt(P["Vc"], torch.bfloat16), _t(P["tables"], torch.int32), P["max_blocks"], run_start,
            _t([s for s, _ in runs], torch.int32), len(runs), max(n for _, n in runs), nh, nkv, hd, 1.0 / math.sqrt(hd))
    a = torch.full((R, nh * hd), 3.0, dtype=torch.bfloat16, device=DEV)
    b = torch.full((R, nh * hd), 5.0, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(q_rot, a, *args)
    ops.attention_prefill(q_plain, b, *args, cos_sin=table)
    assert torch.equal(a, b)
    # and the rotation itself moved something: unrotated queries give another result
    c = torch.full((R, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(q_plain, c, *args)
    assert not torch.equal(a, c)
    # the k heads alone: skip_q leaves q as it was and still rotates and stores the keys
    fused = torch.zeros(R, (nh + 2 * nkv) * hd, dtype=torch.bfloat16, device=DEV)
    fused[:, :nh * hd] = q_plain
    fused[:, nh * hd:] = torch.randn(R, 2 * nkv * hd, device=DEV).to(torch.bfloat16)
    both, only_k = fused.clone(), fused.clone()
    ops.rope_cache(both, nh, nkv, hd, cos_sin=table)
    ops.rope_cache(only_k, nh, nkv, hd, cos_sin=table, skip_q=True)
    assert torch.equal(only_k[:, :nh * hd], fused[:, :nh * hd])
    assert torch.equal(only_k[:, nh * hd:], both[:, nh * hd:])


def test_prefill_attention_is_causal_at_tile_and_page_edges(ops):
    """A huge key at position t must be seen by rows t, t+1, .. and by no row before it."""
    rng = np.random.default_rng(50)
    nh, nkv, hd, B = 4, 2, 64, 16
    runs = [(0, 200)]
    for t in (0, 15, 16, 63, 64, 65, 127, 128, 199):
        P = _runs_problem(rng, runs, nh, nkv, hd, B)
        P["Q"][:, 1] = 0.0
        P["Q"][:, 1, 9] = 30.0
        kvec = np.zeros(hd)
        kvec[9] = 30.0
        P["Kl"][0][t, 0] = kvec
        P["Kc"][P["tables"][0, t // B], 0, t % B] = kvec
        got = _run_prefill(ops, P, runs, nh, nkv, hd, scale=1.0)
        np.testing.assert_allclose(got[t:, 1], np.broadcast_to(P["Vl"][0][t, 0], got[t:, 1].shape), atol=2e-2)
        if t > 0:
            ref = _ref_attention(P, nh, nkv, hd, scale=1.0)
            np.testing.assert_allclose(got[:t, 1], ref[:t, 1], atol=2e-2)
            assert np.abs(got[t - 1, 1] - P["Vl"][0][t, 0]).max() > 0.1


def test_prefill_attention_long_prompt(ops):
    rng = np.random.default_rng(51)
    nh, nkv, hd, B = 8, 2, 64, 16
    runs = [(0, 1500), (1000, 300)]
    P = _runs_problem(rng, runs, nh, nkv, hd, B)
    got = _run_prefill(ops, P, runs, nh, nkv, hd)
    # a launch this narrow cuts contexts into segments of keys that are merged afterwards: rows
    # around the cuts (and around multiples of 512, where cuts lie in other launches), a tile that a cut goes through (the second run starts at 1000), tile edges
    # (little work at head_dim 64: workgroups of 64 rows, and with twice the workgroups segments of 1,024 keys)
    assert ops.attention_prefill_tile_rows(1800, nh, hd, 1500, 1500, 2) == 64 and ops.attention_prefill_segment(1800, nh, hd, 1500, 1500, 2) == 1024
    rows = [0, 1, 63, 64, 511, 512, 513, 700, 1023, 1024, 1025, 1151, 1152, 1499, 1500, 1523, 1524, 1535, 1536, 1627, 1628, 1799]
    ref = np.zeros((len(rows), nh, hd))
    for k, r in enumerate(rows):
        s, c = P["row_seq"][r], P["ctx"][r]
        ref[k] = plain.attention(P["Q"][r:r + 1], P["Kl"][s][:c], P["Vl"][s][:c], [c - 1], np.arange(c), 1.0 / math.sqrt(hd))[0]
    np.testing.assert_allclose(got[rows], ref, atol=1e-2, rtol=0)


def test_prefill_attention_three_segments_far_key(ops):
    """A row deep in the fifth segment of keys must still find one outstanding key of the first."""
    rng = np.random.default_rng(52)
    nh, nkv, hd, B = 4, 1, 128, 16
    runs = [(0, 2300)]
    P = _runs_problem(rng, runs, nh, nkv, hd, B)
    far = 5
    P["Q"][2200:, 2] = 0.0
    P["Q"][2200:, 2, 11] = 30.0
    kvec = np.zeros(hd)
    kvec[11] = 30.0
    P["Kl"][0][far, 0] = kvec
    P["Kc"][P["tables"][0, far // B], 0, far % B] = kvec
    got = _run_prefill(ops, P, runs, nh, nkv, hd, scale=1.0)
    np.testing.assert_allclose(got[2200:, 2], np.broadcast_to(P["Vl"][0][far, 0], got[2200:, 2].shape), atol=2e-2)
    rows = [2047, 2048, 2175, 2176, 2299]
    ref = np.zeros((len(rows), nh, hd))
    for k, r in enumerate(rows):
        c = P["ctx"][r]
        ref[k] = plain.attention(P["Q"][r:r + 1], P["Kl"][0][:c], P["Vl"][0][:c], [c - 1], np.arange(c), 1.0)[0]
    np.testing.assert_allclose(got[rows], ref, atol=1e-2, rtol=0)


@pytest.mark.parametrize("B", [16, 8, 128])
def test_prefill_attention_longer_segments_when_the_launch_is_wide(ops, B):
    """The wider a launch (tiles x heads x sequences), the longer its segments of keys; one that fills
    the chip by itself is not cut at all.  Here 64 heads over a long context give workgroups of 128
    rows and segments of 2,048 keys: rows on both sides of the cut at 6,144, and a far key of the
    first segment."""
    rng = np.random.default_rng(53)
    nh, nkv, hd = 64, 8, 64
    runs = [(6000, 256)]
    assert ops.attention_prefill_tile_rows(256, nh, hd, 6256, 256, 1) == 128 and ops.attention_prefill_segment(256, nh, hd, 6256, 256, 1) == 2048
    assert ops.attention_prefill_tile_rows(2048, 32, 64, 2048, 2048, 1) == 64 and ops.attention_prefill_segment(2048, 32, 64, 2048, 2048, 1) == 2048
    assert ops.attention_prefill_tile_rows(3072, 32, 64, 3072, 3072, 1) == 128 and ops.attention_prefill_tile_rows(2048, 32, 128, 2048, 2048, 1) == 128
    assert ops.attention_prefill_segment(4096, 32, 64, 32768, 4096, 1) == 16384 and ops.attention_prefill_segment(128, 4, 128, 32768, 128, 1) == 512
    P = _paged_problem(rng, [s + n for s, n in runs], nh, nkv, hd, B, all_rows=False)
    R = sum(n for _, n in runs)
    Q = _bf16_grid(rng.normal(size=(R, nh, hd)))
    far, seq, head = 40, 0, 9                                   # kv head 1
    Q[100:, head] = 0.0
    Q[100:, head, 3] = 30.0
    kvec = np.zeros(hd)
    kvec[3] = 30.0
    P["Kl"][seq][far, 1] = kvec
    P["Kc"][P["tables"][seq, far // B], 1, far % B] = kvec
    P["Q"], P["R"] = Q, R
    got = _run_prefill(ops, P, runs, nh, nkv, hd, scale=1.0)
    np.testing.assert_allclose(got[100:, head], np.broadcast_to(P["Vl"][seq][far, 1], (R - 100, hd)), atol=2e-2)
    for r in (0, 127, 128, 143, 144, 145, 255):                # the cut lies between positions 6143 and 6144
        pos = runs[0][0] + r
        ref = plain.attention(Q[r:r + 1], P["Kl"][0][:pos + 1], P["Vl"][0][:pos + 1], [pos], np.arange(pos + 1), 1.0)[0]
        np.testing.assert_allclose(got[r], ref, atol=1e-2, rtol=0, err_msg=f"row {r}")


# ------------------------------------- products of at most 8 rows with the norm folded in
def _folded_reference(a, wo, x, g, eps, w2):
    """What the producer and the consumer compute, in float64 with the same rounding points:
    x += round(a wo^T); xg = round(g round(x)); y = round((xg w2^T) rsqrt(mean x^2 + eps))."""
    x_new = x + _bf16_grid(a @ wo.T)
    xg = _bf16_grid(g * _bf16_grid(x_new))
    rstd = 1.0 / np.sqrt((x_new ** 2).mean(-1, keepdims=True) + eps)
    return x_new, xg, (xg @ w2.T) * rstd


@pytest.mark.parametrize("M", [1, 3, 5, 8])
@pytest.mark.parametrize("H,K,N2", [(2048, 2048, 2560), (2048, 5632, 512), (128, 64, 48), (320, 192, 32), (2048, 2112, 4128)])
def test_products_with_the_norm_folded_in(ops, M, H, K, N2):
    """Producer (residual add + the norm's preparation in the epilogue) and consumer (the norm's scale on
    the finished sums) against the same arithmetic in float64, and against the reference's own form of
    the norm, whose two roundings fall at other places (kernels.cu:34-49): equal up to bfloat16 rounding.
    Widths that are no power of two, K slices of unequal length, fewer rows than a tile holds."""
    rng = np.random.default_rng(M * 13 + H + K)
    a = _bf16_grid(rng.normal(size=(M, K)))
    wo = _bf16_grid(rng.normal(size=(H, K)) * 0.05)
    x = (rng.normal(size=(M, H)) * 2).astype(np.float32).astype(np.float64)
    g = _bf16_grid(1 + 0.1 * rng.normal(size=H))
    w2 = _bf16_grid(rng.normal(size=(N2, H)) * 0.05)
    eps = 1e-5
    x_new, xg_ref, y_ref = _folded_reference(a, wo, x, g, eps, w2)

    at, wot, w2t = _t(a, torch.bfloat16), _t(wo, torch.bfloat16), _t(w2, torch.bfloat16)
    xt = _t(x, torch.float32)
    xg = torch.full((16, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    ss = torch.full((16, H // 8), float("nan"), dtype=torch.float32, device=DEV)
    normed_buf = torch.zeros(M, H, dtype=torch.bfloat16, device=DEV)
    product = ops.PendingProduct(at, wot, torch.zeros(M, H, dtype=torch.bfloat16, device=DEV))
    assert ops.gemm8_supported(M, H, K) and ops.gemm8_supported(M, N2, H)
    h = ops.gemm_residual_norm(product, xt, _t(g, torch.bfloat16), eps, xg, ss, normed_buf)
    # the residual stream: a 32-bit sum of x and the rounded product (the product's last bit may fall either way)
    np.testing.assert_allclose(_np(xt), x_new, rtol=0, atol=2 ** -7 * np.abs(a @ wo.T).max())
    got_x = _np(xt)
    np.testing.assert_allclose(_np(ss[:M]).sum(-1), (got_x ** 2).sum(-1), rtol=1e-5)
    np.testing.assert_array_equal(_np(xg[:M]), _bf16_grid(g * _bf16_grid(got_x)))
    assert torch.isnan(xg[M:].float()).all() and torch.isnan(ss[M:]).all(), "rows beyond M were written"

    for dtype in (torch.bfloat16, torch.float32):
        y = torch.full((M, N2), float("nan"), dtype=dtype, device=DEV)
        assert ops.gemm(h, w2t, y) is y
        scale = np.abs(y_ref).max()
        np.testing.assert_allclose(_np(y), y_ref, rtol=0, atol=(2 ** -7 if dtype == torch.bfloat16 else 1e-3) * scale)
    # against the reference's form: norm rows rounded as kernels.cu does, then the product
    plain_y = plain.linear(plain.rms_norm(x_new, g, eps, plain.round_bf16), w2)
    np.testing.assert_allclose(_np(y), plain_y, rtol=0, atol=1.5e-2 * np.abs(plain_y).max())
    # the ordinary normed rows are still to be had
    np.testing.assert_allclose(_np(h.materialize()), plain.rms_norm(got_x, g, eps, plain.round_bf16), rtol=2 ** -7, atol=1e-3)


@pytest.mark.parametrize("M", [1, 5, 8])
@pytest.mark.parametrize("H,I", [(2048, 5632), (192, 144), (64, 16), (320, 8192 + 64)])
def test_gate_up_product_with_the_norm_folded_in_applies_swiglu(ops, M, H, I):
    """(the widest case goes through the shared-rows kernel's form of it, which very wide gate/up matrices take)"""
    assert bool(ops.lib().kvcm_gemm_skinny_swiglu_normed_preferred(M, I, H)) == (I > 8192)
    rng = np.random.default_rng(M + H + I)
    x = (rng.normal(size=(M, H)) * 2).astype(np.float32).astype(np.float64)
    g = _bf16_grid(1 + 0.1 * rng.normal(size=H))
    wgu = _bf16_grid(rng.normal(size=(2 * I, H)) * 0.05)
    eps = 1e-6
    # a producer with a zero product leaves x as it is and prepares the norm
    xt = _t(x, torch.float32)
    xg = torch.zeros(16, H, dtype=torch.bfloat16, device=DEV)
    ss = torch.zeros(16, H // 8, dtype=torch.float32, device=DEV)
    zero = ops.PendingProduct(torch.zeros(M, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(H, 64, dtype=torch.bfloat16, device=DEV),
                              torch.zeros(M, H, dtype=torch.bfloat16, device=DEV))
    h = ops.gemm_residual_norm(zero, xt, _t(g, torch.bfloat16), eps, xg, ss, torch.zeros(M, H, dtype=torch.bfloat16, device=DEV))
    np.testing.assert_array_equal(_np(xt), x)
    act = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert ops.gemm_swiglu(h, _t(wgu, torch.bfloat16), act)
    xg_ref = _bf16_grid(g * _bf16_grid(x))
    rstd = 1.0 / np.sqrt((x ** 2).mean(-1, keepdims=True) + eps)
    gu = _bf16_grid((xg_ref @ wgu.T) * rstd)
    want = plain.swiglu(gu, plain.round_bf16)
    got = _np(act)
    assert np.mean(got == want) > 0.97                       # a sum's last bit may fall the other way before rounding
    np.testing.assert_allclose(got, want, rtol=2 ** -6, atol=2e-3)
    # and the reference's form of norm then product then SwiGLU is the same up to rounding
    ref = plain.swiglu(np.concatenate([plain.linear(plain.rms_norm(x, g, eps, plain.round_bf16), wgu[:I], plain.round_bf16),
                                       plain.linear(plain.rms_norm(x, g, eps, plain.round_bf16), wgu[I:], plain.round_bf16)], -1),
                       plain.round_bf16)
    np.testing.assert_allclose(got, ref, rtol=0, atol=2e-2 * max(np.abs(ref).max(), 1e-3))


@pytest.mark.parametrize("M", [1, 6, 8])
def test_small_product_plain_form_and_refusals(ops, M):
    """The same kernel without a norm in front (a tensor in x's place), float32 and bfloat16 results,
    one and two column groups per workgroup; shapes it does not take are refused by the entry."""
    rng = np.random.default_rng(77 + M)
    for N, K in ((4096 + 16, 128), (16400, 64), (48, 320)):
        x = _bf16_grid(rng.normal(size=(M, K)))
        w = _bf16_grid(rng.normal(size=(N, K)) * 0.05)
        for dtype in (torch.bfloat16, torch.float32):
            out = torch.full((M, N), float("nan"), dtype=dtype, device=DEV)
            ops._gemm8(_t(x, torch.bfloat16), _t(w, torch.bfloat16), out, N, False)
            tol = dict(rtol=2 ** -7, atol=1e-3) if dtype == torch.bfloat16 else dict(rtol=0, atol=2e-5 * math.sqrt(K))
            np.testing.assert_allclose(_np(out), plain.linear(x, w), **tol)
    assert not ops.gemm8_supported(9, 2048, 2048) and not ops.gemm8_supported(4, 2044, 2048) and not ops.gemm8_supported(4, 2048, 96)
    assert ops.gemm8_supported(8, 24, 64) and not ops.gemm8_supported(16, 32, 64)      # more than 8 rows: another kernel's
    with pytest.raises(ops.KernelError, match="unsupported shape"):
        ops._gemm8(torch.zeros(9, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(16, 64, dtype=torch.bfloat16, device=DEV),
                   torch.zeros(9, 16, dtype=torch.bfloat16, device=DEV), 16, False)


# ------------------------------------------------ where the order of rounding and multiplying shows
def test_norm_and_swiglu_kernels_round_where_the_reference_rounds(ops):
    """Inputs for which rounding before or after the multiply gives different 16-bit values (and which
    stay clear of rounding boundaries by far more than 32-bit arithmetic can shift them): the kernels
    give the plain functions' bits, element for element (src/cuda/kernels.cu:34-49 and 72-82)."""
    import helpers as H
    r = plain.round_bf16
    x, w = H.norm_rounding_cases()
    want = plain.rms_norm(x, w, 1e-6, r)
    inv = 1.0 / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6)
    assert (want != r(w * x * inv)).mean() > 0.05
    out = torch.zeros(x.shape, dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(_t(x, torch.float32), _t(w, torch.bfloat16), out, 1e-6)
    np.testing.assert_array_equal(_np(out), want)
    # the norm with the pending addition and the gathered form round at the same places
    half = (x / 2).astype(np.float32).astype(np.float64)
    assert np.array_equal(half * 2, x)
    xt = _t(half, torch.float32)
    out2 = torch.zeros_like(out)
    ops.rmsnorm(xt, _t(w, torch.bfloat16), out2, 1e-6, add=_t(half, torch.float32))
    np.testing.assert_array_equal(_np(out2), want)
    rows = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
    out3 = torch.zeros(2, x.shape[1], dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(_t(x, torch.float32), _t(w, torch.bfloat16), out3, 1e-6, rows=rows)
    np.testing.assert_array_equal(_np(out3), want[[2, 0]])

    g, u = H.swiglu_rounding_cases()
    rows_, I = g.shape
    act_want = plain.swiglu(np.concatenate([g, u], -1), r)
    silu = g / (1.0 + np.exp(-g))
    assert (act_want != r(silu * u)).mean() > 0.05
    act = torch.zeros(rows_, I, dtype=torch.bfloat16, device=DEV)
    ops.swiglu(_t(np.concatenate([g, u], -1), torch.bfloat16), act)
    np.testing.assert_array_equal(_np(act), act_want)
    # the same values as the result of a product: row m of X picks column m of the weights, so that the
    # sums are the chosen gate and up values themselves; the products' SwiGLU epilogues round alike
    K = 64
    X = np.zeros((rows_, K))
    X[np.arange(rows_), np.arange(rows_)] = 1.0
    W = np.zeros((2 * I, K))
    W[:I, :rows_] = g.T
    W[I:, :rows_] = u.T
    xt, wt = _t(X, torch.bfloat16), _t(W, torch.bfloat16)
    fused = torch.zeros(rows_, I, dtype=torch.bfloat16, device=DEV)
    ops._gemm8(xt, wt, fused, I, True)                                   # the product of at most 8 rows
    np.testing.assert_array_equal(_np(fused), act_want)
    for M in (rows_, 24):                                                # the product whose waves share the rows
        Xm = np.zeros((M, K))
        Xm[:rows_] = X
        wide = 5632                                                      # wide enough for the one-launch form to be taken
        Wm = np.zeros((2 * wide, K))
        Wm[:I, :] = W[:I]
        Wm[wide:wide + I, :] = W[I:]
        out_m = torch.zeros(M, wide, dtype=torch.bfloat16, device=DEV)
        keep, ops.LIBRARY_GEMM_MIN_ROWS = ops.LIBRARY_GEMM_MIN_ROWS, 0
        try:
            assert ops.gemm_swiglu(_t(Xm, torch.bfloat16), _t(Wm, torch.bfloat16), out_m)
        finally:
            ops.LIBRARY_GEMM_MIN_ROWS = keep
        np.testing.assert_array_equal(_np(out_m)[:rows_, :I], act_want)


# ------------------------------------------------ what a page's previous owner left behind
def _poison_beyond_contexts(P, lens, B):
    """Every key and value slot that no sequence of the problem owns (the tails of last pages, the spare
    pages) gets NaN and Inf: what a reused page may hold when its previous owner's values blew up."""
    owned = np.zeros(P["Kc"].shape[:1] + (B,), dtype=bool)
    for s, c in enumerate(lens):
        for t in range(c):
            owned[P["tables"][s, t // B], t % B] = True
    bad = np.where(np.arange(owned.size).reshape(owned.shape) % 2 == 0, np.nan, np.inf)
    for cache in (P["Kc"], P["Vc"]):
        for h in range(cache.shape[1]):
            cache[:, h][~owned] = np.broadcast_to(bad[~owned][:, None], cache[:, h][~owned].shape)
    assert (~owned).sum() > 20


@pytest.mark.parametrize("nh,nkv,hd,B", [(8, 2, 64, 16), (6, 2, 128, 32), (32, 4, 64, 8)])
def test_stale_values_past_a_context_do_not_reach_the_output(ops, nh, nkv, hd, B):
    """Probabilities of slots past a context's end are zero, but zero times a stale NaN or Inf is not:
    the matrix-core kernels cut such slots out of their value pieces.  All four attention kernels."""
    rng = np.random.default_rng(nh + B)
    lens = [700, 257, 33, 1, 250, 511, 9]
    P = _paged_problem(rng, lens, nh, nkv, hd, B, all_rows=False)
    ref = _ref_attention(P, nh, nkv, hd)
    _poison_beyond_contexts(P, lens, B)
    R = P["R"]
    scale = 1.0 / math.sqrt(hd)
    kc, vc = _t(P["Kc"], torch.bfloat16), _vt(P["Vc"], torch.bfloat16)
    assert torch.isnan(vc.float()).any() and torch.isinf(kc.float()).any()
    tables, row_seq, ctx = _t(P["tables"], torch.int32), _t(P["row_seq"], torch.int32), _t(P["ctx"], torch.int32)
    q = _t(P["Q"].reshape(R, nh * hd), torch.bfloat16)

    generic = torch.zeros(R, nh * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention(q, generic, kc, vc, tables, P["max_blocks"], row_seq, ctx, nh, nkv, hd, scale)
    partitioned = torch.zeros_like(generic)
    scratch = torch.zeros(ops.attention_decode_scratch(R, nh, hd, 1024), dtype=torch.float32, device=DEV)
    ops.attention_decode(q, partitioned, kc, vc, tables, P["max_blocks"], row_seq, ctx, nh, nkv, hd, scale, 1024, scratch)
    fused = torch.zeros_like(generic)
    qkv = torch.zeros(R, (nh + 2 * nkv) * hd, dtype=torch.bfloat16, device=DEV)
    qkv[:, :nh * hd] = q
    ops.attention_decode_fused(qkv, fused, kc, vc, tables, P["max_blocks"], row_seq, ctx, nh, nkv, hd, scale, max_context=1024)
    for name, out in (("generic", generic), ("partitioned", partitioned), ("fused", fused)):
        got = _np(out).reshape(R, nh, hd)
        assert np.isfinite(got).all(), name
        np.testing.assert_allclose(got, ref, atol=1e-2, rtol=0, err_msg=name)

    # runs of positions whose last row lies in the middle of a group of 8 slots and of a page
    runs = [(0, 130), (77, 2), (200, 51), (15, 64), (0, 3)]
    Pr = _runs_problem(rng, runs, nh, nkv, hd, B)
    want = _ref_attention(Pr, nh, nkv, hd)
    _poison_beyond_contexts(Pr, [s + n for s, n in runs], B)
    got = _run_prefill(ops, Pr, runs, nh, nkv, hd)
    assert np.isfinite(got).all()
    np.testing.assert_allclose(got, want, atol=1.5e-2, rtol=0)


def test_dependencies_inside_one_launch_hand_data_over_and_every_wait_is_bounded(ops):
    """The probe kernels behind ``kvkernel --sync``: workgroups of one launch meet at a counter and read what
    the others left past the caches (no wrong value, nobody gives up); split sums added by the last
    workgroup to arrive equal those a second launch adds; and a wait that cannot end (the host
    names one arrival more than the launch has workgroups, and a limit of eight polls) ends all the same: every
    workgroup raises the flag and leaves."""
    flags = torch.zeros(2, dtype=torch.int32, device=DEV)
    data = torch.zeros(2 * 64 * 256, dtype=torch.float32, device=DEV)
    counter = torch.zeros(1, dtype=torch.int32, device=DEV)
    ops.probe_barrier(data, counter, flags, 64, 5)
    assert flags.tolist() == [0, 0] and int(counter) == 5 * 64
    S, tiles = 8, 40
    partials = torch.zeros(S * tiles * 1024, dtype=torch.float32, device=DEV)
    counters = torch.zeros(tiles, dtype=torch.int32, device=DEV)
    a, b = torch.zeros(tiles * 1024, dtype=torch.float32, device=DEV), torch.zeros(tiles * 1024, dtype=torch.float32, device=DEV)
    ops.probe_sums(partials, counters, a, S, tiles, True, flags)
    ops.probe_sums(partials, counters, a, S, tiles, True, flags)          # the counters were left at zero
    ops.probe_sums(partials, counters, b, S, tiles, False, flags)
    assert torch.equal(a, b) and float(a.view(tiles, 256, 4)[3, 0, 0]) == S * (S + 1) / 2 and flags.tolist() == [0, 0]
    assert int(counters.abs().sum()) == 0
    # the barrier waits for one arrival more than the launch has workgroups: every workgroup polls eight
    # times, gives up in the first round, and the launch ends
    counter.zero_()
    ops.probe_barrier(data, counter, flags, 64, 3, spin_cap=8, awaited=65)
    torch.cuda.synchronize()
    assert flags.tolist() == [64, 0] and int(counter) == 64
