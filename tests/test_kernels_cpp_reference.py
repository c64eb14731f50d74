"""Each HIP kernel beside its plain C++ reference (csrc/ref/reference.cpp: one loop nest per operation,
double precision inside, no GPU): the same arrays go through both, at sizes other than the engine's and
other than those of tests/test_kernels.py.  bfloat16 inputs are made of values that bfloat16 holds, so
that both sides compute on the same numbers and differ by the kernel's own rounding alone."""
import ctypes
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

F, I32 = ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_int)
TOL = {torch.float32: 3e-6, torch.bfloat16: 8e-3}


@pytest.fixture(scope="module")
def ref():
    from burn_lm_amd.csrc import build
    return ctypes.CDLL(build.ensure_ref_built(verbose=False))


@pytest.fixture(scope="module")
def ops():
    from burn_lm_amd.csrc import ops
    ops.library()
    return ops


def fp(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(F)


def ip(a):
    assert a.dtype == np.int32 and a.flags.c_contiguous
    return a.ctypes.data_as(I32)


def held(shape, g, scale=1.0):
    """float32 values that bfloat16 holds exactly."""
    return (torch.randn(*shape, generator=g) * scale).bfloat16().float()


def rel(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.abs(got - want).max() / max(1e-30, np.abs(want).max()))


def paged(g, lens, nkv, hd, n_pages=24, page=64):
    """Random key and value planes (in the kernels' layouts) and a scrambled page table for sequences of these lengths."""
    perm = torch.randperm(n_pages, generator=g).tolist()
    width = max((n + page - 1) // page for n in lens)
    table = np.full((len(lens), width), -1, dtype=np.int32)
    for b, n in enumerate(lens):
        for j in range((n + page - 1) // page):
            table[b, j] = perm.pop()
    k = held((n_pages, nkv, page, hd), g)
    v = held((n_pages, nkv, hd, page), g)
    return k, v, table


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_gather_and_norm(ops, ref, dtype):
    g = torch.Generator().manual_seed(31)
    V, D, T = 77, 200, 9
    table = held((V, D), g)
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    want = np.zeros((T, D), dtype=np.float32)
    ref.ref_embed_gather(fp(table.numpy()), ip(ids.numpy()), fp(want), T, D)
    got = torch.empty(T, D, dtype=torch.float32, device="cuda")
    ops.embed_gather(table.to(dtype).cuda(), ids.cuda(), got)
    assert np.array_equal(got.cpu().numpy(), want)
    # h += three planes; norm of the rows 5, 0, 5
    h = torch.randn(T, D, generator=g)
    planes = torch.randn(3, T, D, generator=g) * 0.3
    gamma = held((D,), g) + 1
    rows = torch.tensor([5, 0, 5], dtype=torch.int32)
    for use_rows, write_h in ((False, True), (True, False)):
        h_ref, out_ref = h.numpy().copy(), np.zeros((3 if use_rows else T, D), dtype=np.float32)
        ref.ref_add_rmsnorm(fp(h_ref), fp(planes.numpy()), 3, T * D, fp(gamma.numpy()), fp(out_ref),
                            ip(rows.numpy()) if use_rows else None, out_ref.shape[0], D, ctypes.c_float(1e-6), int(write_h))
        h_gpu = h.clone().cuda()
        out = torch.empty(out_ref.shape, dtype=dtype, device="cuda")
        ops.add_rmsnorm(h_gpu, planes.cuda(), gamma.to(dtype).cuda(), 1e-6, out, rows=rows.cuda() if use_rows else None, write_h=write_h)
        assert rel(h_gpu.cpu().numpy(), h_ref) <= 3e-6
        assert rel(out.float().cpu().numpy(), out_ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pairing", [0, 1])
def test_rope_kv_write(ops, ref, dtype, pairing):
    g = torch.Generator().manual_seed(32)
    nh, nkv, hd, page = 7, 7, 48, 64
    lens = [70, 3, 129]
    k0, v0, table = paged(g, lens, nkv, hd)
    pos = np.array([69, 68, 2, 128, 0, 64], dtype=np.int32)
    seq = np.array([0, 0, 1, 2, -1, 2], dtype=np.int32)
    T = len(pos)
    qkv = held((T, (nh + 2 * nkv) * hd), g)
    freqs = 10000.0 ** (-np.arange(0, hd, 2) / hd)
    ang = np.arange(200)[:, None] * freqs[None, :]
    cs = np.stack([np.cos(ang), np.sin(ang)], -1).astype(np.float32)
    q_ref, k_ref, v_ref = qkv.numpy().copy(), k0.numpy().copy(), v0.numpy().copy()
    ref.ref_rope_kv_write(fp(q_ref), ip(pos), ip(seq), ip(table), table.shape[1], fp(cs), fp(k_ref), fp(v_ref), page, T, nh, nkv, hd, pairing)
    q_gpu, k_gpu, v_gpu = qkv.to(dtype).cuda(), k0.to(dtype).cuda(), v0.to(dtype).cuda()
    ops.rope_kv_write(q_gpu, torch.from_numpy(pos).cuda(), torch.from_numpy(seq).cuda(), torch.from_numpy(table).cuda(),
                      torch.from_numpy(cs).cuda(), k_gpu, v_gpu, page, nh, nkv, hd, pairing)
    live = seq >= 0
    nq = nh * hd
    assert rel(q_gpu.float().cpu().numpy()[live][:, :nq], q_ref[live][:, :nq]) <= TOL[dtype]
    assert rel(k_gpu.float().cpu().numpy(), k_ref) <= TOL[dtype] and rel(v_gpu.float().cpu().numpy(), v_ref) <= TOL[dtype]


@pytest.mark.parametrize("kind,nh,nkv,hd,window", [("generic32", 6, 2, 40, 0), ("generic", 6, 2, 40, 0), ("generic", 3, 3, 24, 50),
                                                   ("decode", 12, 4, 48, 0), ("decode", 4, 1, 112, 90), ("prefill", 10, 5, 80, 0),
                                                   ("prefill", 2, 2, 16, 70), ("prefill32", 6, 3, 96, 0), ("prefill32", 9, 3, 32, 70),
                                                   ("prefill32", 4, 1, 128, 0)])
def test_attention(ops, ref, kind, nh, nkv, hd, window, monkeypatch):
    """The generic kernel (float32 and bfloat16), the matrix-core decode kernel with cut key ranges and the
    matrix-core prefill kernels (16 and 32 queries per wavefront): one C++ loop nest is the reference of all."""
    g = torch.Generator().manual_seed(33)
    queries = 16
    if kind == "prefill32":     # the form with 32 queries per wavefront, which a caller picks for steps of many blocks only
        queries, kind = 32, "prefill"
    dtype = torch.float32 if kind == "generic32" else torch.bfloat16
    page, scale = 64, 1.0 / math.sqrt(hd)
    lens = [200, 65, 7]
    k, v, table = paged(g, lens, nkv, hd)
    if kind == "prefill":       # the last tokens of each sequence, packed
        new = [60, 65, 7]
        pos = np.concatenate([np.arange(n - m, n) for n, m in zip(lens, new)]).astype(np.int32)
        seq = np.concatenate([np.full(m, b) for b, m in enumerate(new)]).astype(np.int32)
        cu = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    else:                       # one token each, and one of no sequence
        pos = np.array([199, 64, 6, 0], dtype=np.int32)
        seq = np.array([0, 1, 2, -1], dtype=np.int32)
    T = len(pos)
    stride = (nh + 2 * nkv) * hd
    q = held((T, stride), g)
    want = np.zeros((T, nh * hd), dtype=np.float32)
    ref.ref_attention(fp(q.numpy()), stride, fp(want), ip(pos), ip(seq), ip(table), table.shape[1], fp(k.numpy()), fp(v.numpy()),
                      page, T, nh, nkv, hd, ctypes.c_float(scale), window)
    dev = lambda a: (torch.from_numpy(a) if isinstance(a, np.ndarray) else a).cuda()
    out = torch.full((T, nh * hd), 7.0, dtype=dtype, device="cuda")
    args = (dev(q.to(dtype)), stride, out, dev(pos))
    if kind.startswith("generic"):
        ops.attn_paged(*args, dev(seq), dev(table), dev(k.to(dtype)), dev(v.to(dtype)), page, nh, nkv, hd, scale, window, 3)
    elif kind == "decode":
        assert ops.attn_decode_supported(dtype, hd, page)
        ops.attn_decode(*args, dev(seq), dev(table), dev(k.to(dtype)), dev(v.to(dtype)), page, nh, nkv, hd, scale, window, 2)
    else:
        assert ops.attn_prefill_mfma_supported(dtype, hd, page)
        ops.attn_prefill_mfma(*args, dev(cu), dev(table), dev(k.to(dtype)), dev(v.to(dtype)), page, len(lens), max(new), nh, nkv, hd, scale, window,
                              queries=queries)
    assert rel(out.float().cpu().numpy(), want) <= (1e-5 if dtype == torch.float32 else 1.2e-2)


def test_products_and_gating(ops, ref):
    """Every matrix product kernel against one C++ loop nest: the tiled float product, the skinny float
    product, the matrix-core skinny product (plain, gated, in K-groups), the matrix-core product for many
    rows (plain and gated), the gating kernel, and the resident feed-forward kernel."""
    g = torch.Generator().manual_seed(34)
    M, N, K, I = 6, 150, 328, 80
    A, W = held((M, K), g), held((N, K), g, 0.1)
    want = np.zeros((M, N), dtype=np.float32)
    ref.ref_linear(fp(A.numpy()), fp(W.numpy()), fp(want), M, N, K)
    out = torch.empty(M, N, device="cuda")
    assert rel(ops.gemm_tiled(A.cuda(), W.cuda(), out).cpu().numpy(), want) <= 3e-6
    assert rel(ops.gemv_skinny(A.cuda(), W.cuda(), torch.empty(M, N, device="cuda")).cpu().numpy(), want) <= 3e-6
    Ab, Wb = A.bfloat16().cuda(), W.bfloat16().cuda()
    assert rel(ops.gemv_mfma(Ab, ops.pack_weight(Wb), torch.empty(M, N, device="cuda"), K).cpu().numpy(), want) <= 3e-6
    planes = ops.gemv_mfma(Ab, ops.pack_weight(Wb), torch.empty(3, M, N, device="cuda"), K)
    assert rel(planes.sum(0).cpu().numpy(), want) <= 3e-6
    # many rows on the matrix cores
    M2 = 210
    A2 = held((M2, K), g)
    want2 = np.zeros((M2, N), dtype=np.float32)
    ref.ref_linear(fp(A2.numpy()), fp(W.numpy()), fp(want2), M2, N, K)
    assert rel(ops.gemm_mfma(A2.bfloat16().cuda(), Wb, torch.empty(M2, N, device="cuda")).cpu().numpy(), want2) <= 3e-6
    # gated: [gate rows; up rows]
    Wg = held((2 * I, K), g, 0.08)
    wantg = np.zeros((M, I), dtype=np.float32)
    ref.ref_gated_linear(fp(A.numpy()), fp(Wg.numpy()), fp(wantg), M, I, K)
    got = ops.gemv_mfma(Ab, ops.pack_weight(Wg.bfloat16().cuda(), gated=True), torch.empty(M, I, dtype=torch.bfloat16, device="cuda"), K, gated=True)
    assert rel(got.float().cpu().numpy(), wantg) <= 8e-3
    wantg2 = np.zeros((M2, I), dtype=np.float32)
    ref.ref_gated_linear(fp(A2.numpy()), fp(Wg.numpy()), fp(wantg2), M2, I, K)
    got = ops.gemm_mfma(A2.bfloat16().cuda(), Wg.bfloat16().cuda(), torch.empty(M2, I, dtype=torch.bfloat16, device="cuda"), gated=True)
    assert rel(got.float().cpu().numpy(), wantg2) <= 8e-3
    gu = held((M2, 2 * I), g)
    wants = np.zeros((M2, I), dtype=np.float32)
    ref.ref_swiglu(fp(gu.numpy()), fp(wants), M2, I)
    assert rel(ops.swiglu(gu.cuda(), torch.empty(M2, I, device="cuda")).cpu().numpy(), wants) <= 3e-6


def test_argmax_and_sample(ops, ref):
    g = torch.Generator().manual_seed(35)
    R, V, ld = 11, 3001, 3008
    logits = torch.randn(R, ld, generator=g) * 2
    logits[3, 100] = logits[3, 2000] = 30.0     # a tie: the lower index
    logits[:, V:] = 99.0                          # beyond the vocabulary
    want = np.zeros(R, dtype=np.int32)
    ref.ref_argmax(fp(logits.numpy()), ip(want), R, V, ld)
    assert ops.argmax(logits.cuda()[:, :V]).cpu().numpy().tolist() == want.tolist() and want[3] == 100
    u = torch.rand(R, generator=g)
    for temperature, top_p in ((0.7, 1.0), (1.3, 0.9), (0.5, 0.35)):
        ref.ref_sample(fp(logits.numpy()), fp(u.numpy()), ip(want), R, V, ld, ctypes.c_float(temperature), ctypes.c_float(top_p))
        got = ops.sample(logits.cuda()[:, :V], u.cuda(), temperature, top_p).cpu().numpy()
        # a draw that falls within float rounding of a boundary of the cumulative distribution may go to the neighbour
        assert (got == want).mean() >= 0.9, (temperature, top_p, got.tolist(), want.tolist())
