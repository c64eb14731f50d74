"""Each HIP kernel alone against a plain float32 / float64 torch expression of the same
operation, at sizes other than the engine's (widths and vocabularies that are no powers of two,
odd head counts, several head sizes), in float32 and bfloat16."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# one rounding to the storage type, relative to the largest value of the row
EPS = {"float32": 2e-6, "bfloat16": 6e-3}


@pytest.fixture(scope="module")
def ops():
    from burn_lm_amd.csrc import ops
    ops.library()
    return ops


def dev(t):
    return t.to("cuda")


def close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= tol, f"relative error {err:.3g} > {tol}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed_gather(ops, dtype):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(1000, 200, generator=g).to(DT[dtype])
    ids = torch.tensor([0, 999, 5, 5, 123], dtype=torch.int32)
    h = torch.empty(5, 200, dtype=torch.float32, device="cuda")
    ops.embed_gather(dev(table), dev(ids), h)
    assert torch.equal(h.cpu(), table[ids.long()].float())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed_gather_with_tokens_left_on_the_device(ops, dtype):
    """Rows whose source row is >= 0 take their token from the array whose address is in the cell;
    the cell is changed between two calls, as between two replays; a token outside the table gives NaN."""
    g = torch.Generator().manual_seed(0)
    table = torch.randn(333, 72, generator=g).to(DT[dtype])
    ids = dev(torch.tensor([7, 8, 9, 10, 11, 12], dtype=torch.int32))
    rows = dev(torch.tensor([2, -1, 0, -1, 1, 2], dtype=torch.int32))
    cell = torch.zeros(1, dtype=torch.int64, device="cuda")
    h = torch.empty(6, 72, dtype=torch.float32, device="cuda")
    for left in ([300, 0, 332], [5, 6, 7, 8]):
        source = dev(torch.tensor(left, dtype=torch.int32))
        cell.fill_(source.data_ptr())
        ops.embed_gather_from(dev(table), ids, rows, cell, h)
        expect = [left[2], 8, left[0], 10, left[1], left[2]]
        assert torch.equal(h.cpu(), table[torch.tensor(expect)].float())
    source = dev(torch.tensor([1, 333, -1], dtype=torch.int32))
    cell.fill_(source.data_ptr())
    ops.embed_gather_from(dev(table), ids, rows, cell, h)
    bad = torch.isnan(h).all(1).cpu().tolist()
    assert bad == [True, False, False, False, True, True] and not torch.isnan(h[1]).any()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("gamma_dtype", ["float32", "bfloat16"])
def test_add_rmsnorm(ops, dtype, gamma_dtype):
    g = torch.Generator().manual_seed(1)
    T, D, eps = 7, 200, 1e-3
    h = torch.randn(T, D, generator=g) * 0.02          # small, so eps matters
    delta = (torch.randn(T, D, generator=g) * 0.02).to(DT[dtype])
    gamma = (1 + 0.3 * torch.randn(D, generator=g)).to(DT[gamma_dtype])

    def ref(v):
        v = v.double()
        return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * gamma.double()

    hd = dev(h.clone())
    out = torch.empty(T, D, dtype=DT[dtype], device="cuda")
    ops.add_rmsnorm(hd, dev(delta), dev(gamma), eps, out)
    summed = h + delta.float()
    assert torch.equal(hd.cpu(), summed), "the residual sum is float32 and written back"
    close(out, ref(summed), EPS[dtype])
    # eps inside the root: leaving it out changes these small rows a lot
    assert float((ref(summed) - summed.double() / summed.double().pow(2).mean(-1, keepdim=True).sqrt() * gamma.double()).abs().max()) > 0.05
    # no delta; rows gathered; h untouched
    hd = dev(h.clone())
    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    out = torch.empty(3, D, dtype=DT[dtype], device="cuda")
    ops.add_rmsnorm(hd, None, dev(gamma), eps, out, rows=dev(rows))
    close(out, ref(h[rows.long()]), EPS[dtype])
    ops.add_rmsnorm(hd, dev(delta), dev(gamma), eps, out, rows=dev(rows), write_h=False)
    close(out, ref(summed[rows.long()]), EPS[dtype])
    assert torch.equal(hd.cpu(), h)


def _rope_ref(x, pos, freqs, pairing):
    """x [T, heads, hd] double; complex multiplication on the pairs."""
    ang = pos.double()[:, None] * freqs[None, :]
    rot = torch.polar(torch.ones_like(ang), ang)[:, None, :]
    hd = x.shape[-1]
    if pairing == "interleaved":
        z = torch.complex(x[..., 0::2], x[..., 1::2]) * rot
        out = torch.empty_like(x)
        out[..., 0::2], out[..., 1::2] = z.real, z.imag
    else:
        z = torch.complex(x[..., : hd // 2], x[..., hd // 2:]) * rot
        out = torch.cat([z.real, z.imag], -1)
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("pairing", ["interleaved", "half"])
@pytest.mark.parametrize("nh,nkv,hd", [(6, 3, 32), (5, 5, 24), (8, 1, 80)])
def test_rope_kv_write(ops, dtype, pairing, nh, nkv, hd):
    from burn_lm_amd.parts.rope import PAIRING, rope_frequencies
    g = torch.Generator().manual_seed(2)
    page, n_pages = 16, 12
    # two sequences: 5 new tokens at positions 30..34 (crossing a page edge), 1 new token at position 3
    positions = torch.tensor([30, 31, 32, 33, 34, 3], dtype=torch.int32)
    token_seq = torch.tensor([0, 0, 0, 0, 0, 1], dtype=torch.int32)
    table = torch.tensor([[7, 2, 9, -1], [4, -1, -1, -1]], dtype=torch.int32)
    T = 6
    qkv = torch.randn(T, (nh + 2 * nkv) * hd, generator=g).to(DT[dtype])
    freqs = torch.from_numpy(rope_frequencies(hd, 500000.0, (8, 1, 4, 32)))
    ang = torch.arange(64).double()[:, None] * freqs[None, :]
    cs = torch.stack([ang.cos(), ang.sin()], -1).float()
    k = torch.full((n_pages, nkv, page, hd), 99.0).to(DT[dtype])
    v = torch.full((n_pages, nkv, hd, page), 99.0).to(DT[dtype])      # values are kept transposed per page
    qd, kd, vd = dev(qkv.clone()), dev(k), dev(v)
    ops.rope_kv_write(qd, dev(positions), dev(token_seq), dev(table), dev(cs), kd, vd, page, nh, nkv, hd,
                      PAIRING[pairing])
    x = qkv.double()
    q_ref = _rope_ref(x[:, : nh * hd].reshape(T, nh, hd), positions, freqs, pairing)
    k_ref = _rope_ref(x[:, nh * hd: (nh + nkv) * hd].reshape(T, nkv, hd), positions, freqs, pairing)
    v_ref = x[:, (nh + nkv) * hd:].reshape(T, nkv, hd)
    close(qd[:, : nh * hd].reshape(T, nh, hd), q_ref, EPS[dtype])
    assert torch.equal(qd[:, nh * hd:].cpu(), qkv[:, nh * hd:]), "k and v in the activation buffer stay as they were"
    kc, vc = kd.cpu().double(), vd.cpu().double()
    written = torch.zeros(n_pages, page, dtype=torch.bool)
    for t in range(T):
        p = int(positions[t])
        pg = int(table[int(token_seq[t]), p // page])
        written[pg, p % page] = True
        close(kc[pg, :, p % page], k_ref[t], EPS[dtype])
        assert torch.equal(vc[pg, :, :, p % page], v_ref[t].to(DT[dtype]).double())
    untouched = ~written[:, None, :, None].expand(n_pages, nkv, page, hd)
    assert bool((kc[untouched] == 99).all()), "nothing else is written"
    assert bool((vc.transpose(2, 3)[untouched] == 99).all()), "nothing else is written"
    # a place that reads another's cache rotates q only
    qd2, kd2 = dev(qkv.clone()), dev(k)
    ops.rope_kv_write(qd2, dev(positions), dev(token_seq), dev(table), dev(cs), kd2, dev(v), page, nh, nkv, hd,
                      PAIRING[pairing], write_kv=False)
    assert torch.equal(qd2.cpu(), qd.cpu()) and bool((kd2.cpu() == 99).all())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_swiglu(ops, dtype):
    g = torch.Generator().manual_seed(3)
    T, I = 5, 300
    gu = (torch.randn(T, 2 * I, generator=g) * 3).to(DT[dtype])
    out = torch.empty(T, I, dtype=DT[dtype], device="cuda")
    ops.swiglu(dev(gu), out)
    x = gu.double()
    close(out, torch.nn.functional.silu(x[:, :I]) * x[:, I:], EPS[dtype])


def _attn_ref(q, keys, values, pos, scale, window, n_rep):
    """q [nh, hd]; keys/values [S, nkv, hd] of the whole sequence; query at position pos."""
    lo = max(0, pos - window + 1) if window else 0
    k = keys[lo: pos + 1].double().repeat_interleave(n_rep, 1)
    v = values[lo: pos + 1].double().repeat_interleave(n_rep, 1)
    s = torch.einsum("hd,shd->hs", q.double(), k) * scale
    return torch.einsum("hs,shd->hd", torch.softmax(s, -1), v)


@pytest.mark.parametrize("splits", [1, 2, 5])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (6, 1, 24, 0), (5, 5, 64, 0), (8, 2, 128, 0),
                                               (3, 1, 200, 0), (4, 2, 32, 37), (8, 1, 48, 21), (4, 1, 64, 0)])
def test_attn_paged(ops, dtype, nh, nkv, hd, window, splits):
    """The generic kernel, whole key ranges and ranges cut into pieces that are merged by the last
    wavefront to finish (more pieces than some sequences have chunks of keys: empty pieces).  Head
    sizes up to 128 run the form that stages values through shared memory (groups of four and eight
    heads share one tile of keys and one of values per block), 200 the direct one."""
    ops.attn_paged_init()
    g = torch.Generator().manual_seed(4)
    page, n_pages = 16, 40
    lens = [150, 1, 70]          # cached length of three sequences after this step
    new = [4, 1, 70]             # the last `new` positions are this step's queries
    perm = torch.randperm(n_pages, generator=g).tolist()
    width = 10
    table = torch.full((3, width), -1, dtype=torch.int32)
    keys, values = [], []
    kc = torch.full((n_pages, nkv, page, hd), float("nan"))
    vc = torch.full((n_pages, nkv, hd, page), float("nan"))
    for b, L in enumerate(lens):
        kb = torch.randn(L, nkv, hd, generator=g).to(DT[dtype])
        vb = torch.randn(L, nkv, hd, generator=g).to(DT[dtype])
        if L > 100:   # a far key that the last queries must find: scale it up
            kb[5] *= 6.0
        keys.append(kb); values.append(vb)
        for i in range((L + page - 1) // page):
            pg = perm.pop()
            table[b, i] = pg
            n = min(page, L - i * page)
            kc[pg, :, :n] = kb[i * page: i * page + n].transpose(0, 1).float()
            vc[pg, :, :, :n] = vb[i * page: i * page + n].permute(1, 2, 0).float()
    positions, token_seq = [], []
    for b, (L, n) in enumerate(zip(lens, new)):
        positions += list(range(L - n, L)); token_seq += [b] * n
    positions.append(0); token_seq.append(-1)     # a padding token
    T = len(positions)
    stride = (nh + 2 * nkv) * hd
    qkv = torch.randn(T, stride, generator=g).to(DT[dtype])
    out = torch.full((T, nh * hd), 7.0, dtype=DT[dtype], device="cuda")
    scale = 1.0 / math.sqrt(hd)
    for rep in range(3 if splits > 1 else 1):     # again and again: the counters must come back to zero
        out.fill_(7.0)
        ops.attn_paged(dev(qkv), stride, out, dev(torch.tensor(positions, dtype=torch.int32)),
                       dev(torch.tensor(token_seq, dtype=torch.int32)), dev(table), dev(kc.to(DT[dtype])),
                       dev(vc.to(DT[dtype])), page, nh, nkv, hd, scale, window, splits)
    assert int(ops.arrival_counters("cuda").abs().sum()) == 0
    got = out.cpu().double().reshape(T, nh, hd)
    assert torch.isfinite(got).all(), "a key beyond a sequence's length was read"
    for t in range(T - 1):
        b = token_seq[t]
        want = _attn_ref(qkv[t, : nh * hd].reshape(nh, hd), keys[b], values[b], positions[t], scale, window, nh // nkv)
        close(got[t], want, EPS[dtype] * 2)
    assert bool((got[T - 1] == 0).all()), "a padding token gives zeros"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,window", [(8, 2, 32, 0), (4, 1, 64, 300)])
def test_attn_paged_prompt_of_many_tokens(ops, dtype, nh, nkv, hd, window):
    """A prompt long enough that the generic kernel has blocks in plenty: the four heads of a group then
    share one tile of keys and one of values per block.  Two sequences in one step, pages scattered."""
    ops.attn_paged_init()
    g = torch.Generator().manual_seed(9)
    page, lens = 16, [2200 if nh == 4 else 1100, 130]
    n_pages = sum((L + page - 1) // page for L in lens) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    table = torch.full((2, (max(lens) + page - 1) // page), -1, dtype=torch.int32)
    kc = torch.full((n_pages, nkv, page, hd), float("nan"))
    vc = torch.full((n_pages, nkv, hd, page), float("nan"))
    keys, values, positions, token_seq = [], [], [], []
    for b, L in enumerate(lens):
        kb = torch.randn(L, nkv, hd, generator=g).to(DT[dtype])
        vb = torch.randn(L, nkv, hd, generator=g).to(DT[dtype])
        kb[7] *= 5.0       # an early key that late queries must find (or must not, behind a window)
        keys.append(kb); values.append(vb)
        for i in range((L + page - 1) // page):
            pg = perm.pop()
            table[b, i] = pg
            n = min(page, L - i * page)
            kc[pg, :, :n] = kb[i * page: i * page + n].transpose(0, 1).float()
            vc[pg, :, :, :n] = vb[i * page: i * page + n].permute(1, 2, 0).float()
        positions += list(range(L)); token_seq += [b] * L
    T = len(positions)
    assert T * nh // 4 >= 2048
    stride = (nh + 2 * nkv) * hd
    qkv = torch.randn(T, stride, generator=g).to(DT[dtype])
    out = torch.full((T, nh * hd), 7.0, dtype=DT[dtype], device="cuda")
    scale = 1.0 / math.sqrt(hd)
    ops.attn_paged(dev(qkv), stride, out, dev(torch.tensor(positions, dtype=torch.int32)),
                   dev(torch.tensor(token_seq, dtype=torch.int32)), dev(table), dev(kc.to(DT[dtype])),
                   dev(vc.to(DT[dtype])), page, nh, nkv, hd, scale, window, 1)
    got = out.cpu().double().reshape(T, nh, hd)
    assert torch.isfinite(got).all(), "a key beyond a sequence's length was read"
    rng = torch.Generator().manual_seed(1)
    picks = sorted(set(torch.randint(0, T, (60,), generator=rng).tolist()) | {0, 63, 64, 65, lens[0] - 1, lens[0], T - 1})
    for t in picks:
        b = token_seq[t]
        want = _attn_ref(qkv[t, : nh * hd].reshape(nh, hd), keys[b], values[b], positions[t], scale, window, nh // nkv)
        close(got[t], want, EPS[dtype] * 2)


def _paged_case(g, lens, nkv, hd, page=64, n_pages=40, far_key=None):
    """Random keys and values of several sequences laid out in scrambled pages, NaN everywhere else."""
    perm = torch.randperm(n_pages, generator=g).tolist()
    width = max((L + page - 1) // page for L in lens) + 2
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    keys, values = [], []
    kc = torch.full((n_pages, nkv, page, hd), float("nan"))
    vc = torch.full((n_pages, nkv, hd, page), float("nan"))
    for b, L in enumerate(lens):
        kb = torch.randn(L, nkv, hd, generator=g).bfloat16()
        vb = torch.randn(L, nkv, hd, generator=g).bfloat16()
        if far_key is not None and L > far_key + 60:
            kb[far_key] *= 5.0
        keys.append(kb); values.append(vb)
        for i in range((L + page - 1) // page):
            pg = perm.pop()
            table[b, i] = pg
            n = min(page, L - i * page)
            kc[pg, :, :n] = kb[i * page: i * page + n].transpose(0, 1).float()
            vc[pg, :, :, :n] = vb[i * page: i * page + n].permute(1, 2, 0).float()
    return table, keys, values, kc.bfloat16(), vc.bfloat16()


def test_attn_decode_merge_by_the_last_split_over_many_calls(ops):
    """The splits of a (token, key-value head) are merged by whichever of their blocks finishes last,
    through counters that every call must leave at zero.  A chip-filling case (8 tokens x 8 heads x 16
    splits) run 40 times with fresh queries and a changing number of splits, every result checked; a
    stale partial result or a counter left over from the call before would show."""
    g = torch.Generator().manual_seed(33)
    nh, nkv, hd = 32, 8, 64
    lens = [1500, 1024, 700, 1333, 64, 999, 1471, 300]
    table, keys, values, kc, vc = _paged_case(g, lens, nkv, hd, n_pages=160)
    positions = dev(torch.tensor([L - 1 for L in lens], dtype=torch.int32))
    token_seq = dev(torch.arange(len(lens), dtype=torch.int32))
    table, kc, vc = dev(table), dev(kc), dev(vc)
    stride = (nh + 2 * nkv) * hd
    scale = 1.0 / math.sqrt(hd)
    K = [k.cuda().float() for k in keys]
    V = [v.cuda().float() for v in values]
    counters = ops.arrival_counters("cuda")
    for it in range(40):
        qkv = dev(torch.randn(len(lens), stride, generator=g).bfloat16())
        out = torch.full((len(lens), nh * hd), 7.0, dtype=torch.bfloat16, device="cuda")
        ops.attn_decode(qkv, stride, out, positions, token_seq, table, kc, vc, 64, nh, nkv, hd, scale, 0, (16, 3, 24, 8)[it % 4])
        for b in range(len(lens)):
            q = qkv[b, : nh * hd].float().reshape(nkv, nh // nkv, hd)
            sc = torch.einsum("kgd,lkd->kgl", q, K[b]) * scale
            want = torch.einsum("kgl,lkd->kgd", torch.softmax(sc, -1), V[b]).reshape(nh * hd)
            err = float((out[b].float() - want).abs().max() / want.abs().max())
            assert err <= 1.5e-2, f"call {it} sequence {b}: {err:.3g}"
    assert int(counters.abs().sum()) == 0


@pytest.mark.parametrize("nh,nkv,hd,window,splits", [(4, 2, 16, 0, 3), (6, 1, 32, 0, 1), (5, 5, 64, 0, 4), (8, 2, 128, 0, 16),
                                                      (32, 1, 64, 0, 2), (20, 1, 32, 0, 5), (4, 2, 32, 100, 2),
                                                      (6, 2, 48, 0, 3), (3, 3, 80, 0, 2), (4, 1, 96, 70, 4), (2, 2, 112, 0, 5)])
def test_attn_decode(ops, nh, nkv, hd, window, splits):
    """The matrix-core decode kernel: sequences of very different lengths in one call (one of a single
    key, one that ends exactly at a page edge), scrambled pages with NaN in every unused place, a far
    key that stands out, more splits than some sequences have pages, more than 16 heads to a group,
    a padding token."""
    assert ops.attn_decode_supported(torch.bfloat16, hd) and not ops.attn_decode_supported(torch.bfloat16, 24)
    assert not ops.attn_decode_supported(torch.bfloat16, 144) and not ops.attn_decode_supported(torch.bfloat16, 256)
    assert not ops.attn_decode_supported(torch.float32, hd) and not ops.attn_decode_supported(torch.bfloat16, hd, 16)
    g = torch.Generator().manual_seed(14)
    lens = [403, 1, 64, 17, 130, 65]
    table, keys, values, kc, vc = _paged_case(g, lens, nkv, hd, far_key=2)
    positions = [L - 1 for L in lens] + [0]
    token_seq = list(range(len(lens))) + [-1]
    order = [3, 0, 6, 4, 1, 2, 5]           # the order of the tokens need not be the order of the sequences
    positions = [positions[i] for i in order]; token_seq = [token_seq[i] for i in order]
    T = len(positions)
    stride = (nh + 2 * nkv) * hd
    qkv = torch.randn(T, stride, generator=g).bfloat16()
    out = torch.full((T, nh * hd), 7.0, dtype=torch.bfloat16, device="cuda")
    scale = 1.0 / math.sqrt(hd)
    ops.attn_decode(dev(qkv), stride, out, dev(torch.tensor(positions, dtype=torch.int32)),
                    dev(torch.tensor(token_seq, dtype=torch.int32)), dev(table), dev(kc), dev(vc), 64, nh, nkv, hd,
                    scale, window, splits)
    got = out.cpu().double().reshape(T, nh, hd)
    assert torch.isfinite(got).all(), "a key beyond a sequence's length was read"
    for t in range(T):
        b = token_seq[t]
        if b < 0:
            assert bool((got[t] == 0).all())
            continue
        want = _attn_ref(qkv[t, : nh * hd].reshape(nh, hd), keys[b], values[b], positions[t], scale, window, nh // nkv)
        close(got[t], want, 1.5e-2)


@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (6, 1, 32, 0), (5, 5, 64, 0), (8, 2, 128, 0), (2, 1, 256, 0),
                                               (4, 2, 64, 90), (6, 2, 48, 0), (3, 3, 80, 0), (4, 1, 96, 50), (2, 2, 112, 0)])
@pytest.mark.parametrize("tile", ["16", "32"])
def test_attn_prefill_mfma(ops, nh, nkv, hd, window, tile, monkeypatch):
    """The matrix-core prefill kernel on packed sequences: a whole prompt from position 0 (not a
    multiple of 16 long), a chunk that continues a long past, one token on top of a past that ends at
    a page edge, a single first token; a far key stands out; unused places hold NaN.  Both forms: 16
    queries per wavefront, and 32 (head sizes that are multiples of 32; a caller picks it only for steps
    of many blocks, so it is asked for here)."""
    from burn_lm_amd.csrc.ops import KernelError
    if tile == "32" and (hd % 32 or hd > 128):
        with pytest.raises(KernelError, match="32 queries per wavefront"):
            ops.attn_prefill_mfma(torch.zeros(16, (nh + 2 * nkv) * hd, dtype=torch.bfloat16, device="cuda"), (nh + 2 * nkv) * hd,
                                  torch.zeros(16, nh * hd, dtype=torch.bfloat16, device="cuda"), torch.arange(16, dtype=torch.int32, device="cuda"),
                                  torch.tensor([0, 16], dtype=torch.int32, device="cuda"), torch.zeros(1, 1, dtype=torch.int32, device="cuda"),
                                  torch.zeros(1, nkv, 64, hd, dtype=torch.bfloat16, device="cuda"),
                                  torch.zeros(1, nkv, hd, 64, dtype=torch.bfloat16, device="cuda"), 64, 1, 16, nh, nkv, hd, 0.1, 0, queries=32)
        pytest.skip("the 32-query form takes head sizes 32, 64, 96 and 128 (and says so)")
    assert ops.attn_prefill_mfma_supported(torch.bfloat16, hd) and not ops.attn_prefill_mfma_supported(torch.float32, hd)
    # which form a step takes by itself: 32 queries for several rounds of blocks or a long prompt
    assert ops.attn_prefill_queries(1, 2048, 32, 8, 64, 256) == 16 and ops.attn_prefill_queries(1, 4096, 32, 8, 64, 256) == 32
    assert ops.attn_prefill_queries(4, 2048, 32, 8, 64, 256) == 32 and ops.attn_prefill_queries(1, 65536, 6, 1, 24, 256) == 16
    assert ops.attn_prefill_queries(8, 512, 32, 8, 64, 256) == 16 and ops.attn_prefill_queries(4, 1024, 24, 8, 128, 256) == 16
    assert ops.attn_prefill_queries(32, 512, 32, 8, 64, 256) == 32 and ops.attn_prefill_queries(2, 2048, 32, 8, 128, 256) == 32
    g = torch.Generator().manual_seed(15)
    lens = [150, 333, 65, 1, 40]             # length of each sequence after the step
    new = [150, 70, 1, 1, 33]                # rows this step brings
    table, keys, values, kc, vc = _paged_case(g, lens, nkv, hd, far_key=3)
    positions, cu = [], [0]
    for L, n in zip(lens, new):
        positions += list(range(L - n, L)); cu.append(cu[-1] + n)
    T = len(positions)
    stride = (nh + 2 * nkv) * hd
    qkv = torch.randn(T, stride, generator=g).bfloat16()
    out = torch.full((T, nh * hd), 7.0, dtype=torch.bfloat16, device="cuda")
    scale = 1.0 / math.sqrt(hd)
    ops.attn_prefill_mfma(dev(qkv), stride, out, dev(torch.tensor(positions, dtype=torch.int32)),
                          dev(torch.tensor(cu, dtype=torch.int32)), dev(table), dev(kc), dev(vc), 64, len(lens), max(new),
                          nh, nkv, hd, scale, window, queries=int(tile))
    got = out.cpu().double().reshape(T, nh, hd)
    assert torch.isfinite(got).all(), "a key beyond a sequence's length was read"
    for b in range(len(lens)):
        for t in range(cu[b], cu[b + 1]):
            want = _attn_ref(qkv[t, : nh * hd].reshape(nh, hd), keys[b], values[b], positions[t], scale, window, nh // nkv)
            close(got[t], want, 1.5e-2)


@pytest.mark.parametrize("hd", [64, 48])
def test_attention_over_more_pages_than_a_register_holds_numbers_of(ops, hd):
    """The matrix-core attention kernels keep 64 page numbers of a sequence in one register and load the
    next 64 when a block walks past them.  One sequence of 70 pages with scrambled page numbers: the last
    150 rows of its prompt (both prefill forms), and a decode token over the whole of it uncut and in three
    pieces.  Head size 64 takes its pages straight into shared memory, 48 through registers."""
    g = torch.Generator().manual_seed(16)
    nh, nkv, window = 2, 1, 0
    L, new = 70 * 64 - 21, 150
    table, keys, values, kc, vc = _paged_case(g, [L], nkv, hd, far_key=5, n_pages=75)
    stride = (nh + 2 * nkv) * hd
    scale = 1.0 / math.sqrt(hd)
    positions = list(range(L - new, L))
    qkv = torch.randn(new, stride, generator=g).bfloat16()
    table, kc, vc = dev(table), dev(kc), dev(vc)
    for queries in ((16, 32) if hd % 32 == 0 else (16,)):
        out = torch.full((new, nh * hd), 7.0, dtype=torch.bfloat16, device="cuda")
        ops.attn_prefill_mfma(dev(qkv), stride, out, dev(torch.tensor(positions, dtype=torch.int32)),
                              dev(torch.tensor([0, new], dtype=torch.int32)), table, kc, vc, 64, 1, new, nh, nkv, hd, scale, window,
                              queries=queries)
        got = out.cpu().double().reshape(new, nh, hd)
        assert torch.isfinite(got).all()
        for t in (0, 1, 17, 64, 100, new - 1):
            close(got[t], _attn_ref(qkv[t, : nh * hd].reshape(nh, hd), keys[0], values[0], positions[t], scale, window, nh // nkv), 1.5e-2)
    for splits in (1, 3):
        out = torch.full((1, nh * hd), 7.0, dtype=torch.bfloat16, device="cuda")
        ops.attn_decode(dev(qkv[-1:]), stride, out, dev(torch.tensor([L - 1], dtype=torch.int32)), dev(torch.zeros(1, dtype=torch.int32)),
                        table, kc, vc, 64, nh, nkv, hd, scale, window, splits)
        close(out.cpu().double().reshape(nh, hd),
              _attn_ref(qkv[-1, : nh * hd].reshape(nh, hd), keys[0], values[0], L - 1, scale, window, nh // nkv), 1.5e-2)


def test_attn_paged_refuses_what_it_cannot_do(ops):
    from burn_lm_amd.csrc.ops import KernelError
    z = torch.zeros(1, 3 * 258, device="cuda")
    i = torch.zeros(1, dtype=torch.int32, device="cuda")
    c = torch.zeros(1, 1, 16, 258, device="cuda")
    with pytest.raises(KernelError, match="head_dim 258"):
        ops.attn_paged(z, 3 * 258, torch.zeros(1, 258, device="cuda"), i, i, i.view(1, 1), c, c.transpose(2, 3).contiguous(),
                       16, 1, 1, 258, 1.0)
    with pytest.raises(KernelError, match="cache planes"):
        ops.attn_paged(z, 3 * 258, torch.zeros(1, 258, device="cuda"), i, i, i.view(1, 1), c, c, 16, 1, 1, 258, 1.0)
    with pytest.raises(KernelError, match="GPU only"):
        ops.swiglu(torch.zeros(1, 4), torch.zeros(1, 2))


@pytest.mark.parametrize("a,w,c", [("float32", "float32", "float32"), ("bfloat16", "bfloat16", "bfloat16"),
                                   ("bfloat16", "bfloat16", "float32"), ("bfloat16", "float32", "bfloat16")])
@pytest.mark.parametrize("M,N,K", [(70, 130, 50), (20, 130, 50), (300, 31, 64), (257, 129, 1000), (32, 32, 2)])
def test_gemm_tiled(ops, a, w, c, M, N, K):
    """With fewer than 32 rows or columns the scalar kernel runs, else the matrix cores' float instruction."""
    g = torch.Generator().manual_seed(5)
    A = torch.randn(M, K, generator=g).to(DT[a])
    W = torch.randn(N, K, generator=g).to(DT[w])
    out = torch.empty(M, N, dtype=DT[c], device="cuda")
    ops.gemm_tiled(dev(A), dev(W), out)
    close(out, A.double() @ W.double().T, EPS[c] * 2)
    # rows taken from a wider buffer (unit stride along rows is all that is asked)
    wide = torch.randn(M, K + 14, generator=g).to(DT[a])
    ops.gemm_tiled(dev(wide)[:, :K], dev(W), out)
    close(out, wide[:, :K].double() @ W.double().T, EPS[c] * 2)


def test_float32_product_is_true_32_bit(ops):
    """Operands with 21 significant bits: a matrix mode that rounds its inputs to bfloat16 or to a
    19-bit format returns 16, true float32 returns 16 * (1 + 2^-20); every partial sum is exact."""
    K = 16
    A = torch.full((3, K), 1.0 + 2.0 ** -20)
    W = torch.ones(65, K)
    for fn in (ops.gemm_tiled, ops.gemv_skinny):
        out = torch.empty(3, 65, device="cuda")
        fn(dev(A), dev(W), out)
        assert torch.equal(out.cpu(), torch.full((3, 65), 16.0 + 2.0 ** -16))
    # many rows: the matrix cores' float instruction, which must be as exact
    A, W = torch.full((150, K), 1.0 + 2.0 ** -20), torch.ones(70, K)
    out = torch.empty(150, 70, device="cuda")
    ops.gemm_tiled(dev(A), dev(W), out)
    assert torch.equal(out.cpu(), torch.full((150, 70), 16.0 + 2.0 ** -16))


@pytest.mark.parametrize("M", [8, 17, 64])
def test_float32_product_keeps_its_accuracy_over_a_long_sum(ops, M):
    """8,200 terms of one sign: a single accumulator that takes them one after the other is off by
    5e-6 of the result at the end (measured), sums in two levels or across lanes by a tenth of that."""
    g = torch.Generator().manual_seed(12)
    N, K = 200, 8200
    A = torch.randn(M, K, generator=g).abs()
    W = torch.randn(N, K, generator=g).abs() * 0.05
    out = torch.empty(M, N, device="cuda")
    (ops.gemv_skinny if M <= 8 else ops.gemm_tiled)(dev(A), dev(W), out)
    want = A.double() @ W.double().T
    assert float((out.cpu().double() - want).abs().max() / want.abs().max()) < 1e-6


@pytest.mark.parametrize("dtype,out_dtype", [("float32", "float32"), ("bfloat16", "bfloat16"), ("bfloat16", "float32")])
@pytest.mark.parametrize("M", [1, 2, 3, 5, 8])
def test_gemv_skinny(ops, dtype, out_dtype, M):
    from burn_lm_amd.csrc.ops import KernelError
    g = torch.Generator().manual_seed(6)
    N, K = 1001, 264
    A = torch.randn(M, K, generator=g).to(DT[dtype])
    W = torch.randn(N, K, generator=g).to(DT[dtype])
    out = torch.empty(M, N, dtype=DT[out_dtype], device="cuda")
    ops.gemv_skinny(dev(A), dev(W), out)
    close(out, A.double() @ W.double().T, EPS[out_dtype] * 2)
    with pytest.raises(KernelError, match="multiples of 8"):
        ops.gemv_skinny(dev(A)[:, :260].contiguous(), dev(W)[:, :260].contiguous(), out)
    with pytest.raises(KernelError, match="1..8"):
        ops.gemv_skinny(dev(torch.zeros(9, K).to(DT[dtype])), dev(W), torch.empty(9, N, dtype=DT[out_dtype], device="cuda"))


def test_pack_weight_layout(ops):
    """packed[tile, step, lane, e] = w[tile*16 + lane%16, step*32 + (lane//16)*8 + e], zero padded."""
    N, K = 37, 72
    w = torch.arange(N * K, dtype=torch.float32).reshape(N, K).bfloat16()
    p = ops.pack_weight(dev(w)).cpu().view(3, 3, 64, 8)
    for tile, step, lane, e in [(0, 0, 0, 0), (0, 0, 17, 3), (1, 2, 63, 7), (2, 1, 5, 0), (2, 2, 20, 1), (2, 0, 4, 7)]:
        n, k = tile * 16 + lane % 16, step * 32 + (lane // 16) * 8 + e
        want = float(w[n, k]) if n < N and k < K else 0.0
        assert float(p[tile, step, lane, e]) == want, (tile, step, lane, e)


@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("M,N,K", [(1, 1001, 264), (8, 48, 64), (7, 130, 144), (16, 16, 512), (11, 333, 520),
                                   (8, 257, 2048), (3, 40, 8192), (16, 100, 8200), (5, 31, 14336), (9, 77, 4104),
                                   (2, 9000, 264), (8, 8200, 1024), (6, 100, 4096), (4, 52, 600),
                                   (5, 25000, 1000), (3, 17000, 3080),     # four and five tiles per block, the last block short
                                   (17, 130, 264), (32, 48, 2048), (29, 5000, 2040), (33, 77, 2048), (32, 200, 4096), (20, 1000, 3072), (48, 257, 520),
                                   (47, 16, 64), (49, 300, 1032), (64, 4200, 2048), (61, 40, 136), (35, 20000, 520), (64, 12300, 2048)])
def test_gemv_mfma(ops, out_dtype, M, N, K):
    """Matrix-core skinny product: every way K is cut among wavefronts, tails in N, K and M; above 16
    rows the form with two, three and four row tiles."""
    g = torch.Generator().manual_seed(16)
    A = torch.randn(M, K, generator=g).bfloat16()
    W = torch.randn(N, K, generator=g).bfloat16()
    # make one product term dominate a column so that a wrong operand layout cannot hide in the noise
    W[N // 2, K - 8:] = 40.0
    assert ops.gemv_mfma_supported(M, N, K)
    Wp = ops.pack_weight(dev(W))
    out = torch.full((M, N), 7.0, dtype=DT[out_dtype], device="cuda")
    ops.gemv_mfma(dev(A), Wp, out, K)
    want = A.double() @ W.double().T
    got = out.double().cpu()
    err = ((got - want).abs() / (want.abs() + want.abs().mean())).max()
    assert float(err) <= (2e-5 if out_dtype == "float32" else 8e-3), f"error {float(err):.3g}"
    # rows of a wider buffer, and an output with a row stride
    wide = torch.randn(M, K + 24, generator=g).bfloat16()
    big = torch.zeros(M, N + 5, dtype=DT[out_dtype], device="cuda")
    ops.gemv_mfma(dev(wide)[:, 8:K + 8], Wp, big[:, :N], K)
    close(big[:, :N], wide[:, 8:K + 8].double() @ W.double().T, EPS[out_dtype] * 3)
    assert bool((big[:, N:] == 0).all())


@pytest.mark.parametrize("M,N,K,groups", [(8, 2048, 8192, 2), (3, 100, 2048, 2), (16, 48, 4104, 4), (1, 40, 8192, 8),
                                          (64, 2048, 8192, 4), (24, 100, 8200, 8), (40, 48, 3000, 2), (33, 64, 14336, 8),
                                          (8, 2560, 11008, 3), (5, 72, 2600, 3), (16, 3072, 8192, 6), (2, 56, 12296, 12)])
def test_gemv_mfma_partial_products_are_summed_by_the_norm(ops, M, N, K, groups):
    """K cut into groups handled by different blocks: each plane holds a partial product, their sum is
    the product, and the residual add in front of a norm takes the planes as they are."""
    g = torch.Generator().manual_seed(17)
    A = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    Wp = ops.pack_weight(dev(W))
    planes = torch.full((groups, M, N), 7.0, dtype=torch.float32, device="cuda")
    ops.gemv_mfma(dev(A), Wp, planes, K)
    want = A.double() @ W.double().T
    close(planes.double().sum(0), want, 1e-5)
    steps = (K + 31) // 32
    per = (steps + groups - 1) // groups
    first = A[:, : per * 32].double() @ W[:, : per * 32].double().T
    close(planes[0], first, 1e-5)
    h = torch.randn(M, N, generator=g)
    gamma = (1 + 0.2 * torch.randn(N, generator=g)).bfloat16()
    hd_ = dev(h.clone())
    out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    ops.add_rmsnorm(hd_, planes, dev(gamma), 1e-5, out)
    v = h.double() + planes.double().sum(0).cpu()
    close(hd_, v, 1e-6)
    close(out, v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-5) * gamma.double(), EPS["bfloat16"])
    # gathered rows without writing h back
    rows = torch.tensor([M - 1, 0], dtype=torch.int32)
    hd2 = dev(h.clone())
    out2 = torch.empty(2, N, dtype=torch.bfloat16, device="cuda")
    ops.add_rmsnorm(hd2, planes, dev(gamma), 1e-5, out2, rows=dev(rows), write_h=False)
    assert torch.equal(out2.cpu(), out.cpu()[rows.long()]) and torch.equal(hd2.cpu(), h)


def test_gemv_mfma_says_how_many_blocks_it_launches(ops):
    """The routing counts on it: blocks over all groups and wavefronts per block, only blocks that have a tile."""
    assert ops.gemv_mfma_geometry(8, 2048, 2048, 1) == (128, 4) and ops.gemv_mfma_geometry(8, 2048, 2048, 4) == (512, 4)
    assert ops.gemv_mfma_geometry(8, 3072, 8192, 4) == (384, 4) and ops.gemv_mfma_geometry(8, 3072, 8192, 8) == (512, 2)
    assert ops.gemv_mfma_geometry(8, 4096, 14336, 4) == (256, 7) and ops.gemv_mfma_geometry(1, 128256, 2048, 1) == (501, 4)
    assert ops.gemv_mfma_geometry(40, 2048, 8192, 2) is None and ops.gemv_mfma_geometry(40, 2048, 8192, 4) == (256, 8)
    assert ops.gemv_mfma_geometry(8, 48, 64, 1) == (3, 1)


@pytest.mark.parametrize("M,I,K", [(8, 176, 64), (3, 384, 144), (16, 8, 520), (5, 1000, 2048), (1, 64, 4104), (4, 20000, 2048),
                                   (64, 1000, 2048), (20, 176, 1544), (37, 384, 144), (50, 8, 520), (32, 176, 4096)])
def test_gemv_mfma_gated(ops, M, I, K):
    """The SwiGLU gating in the epilogue of the product that computes gate and up: the packed copy pairs
    every 8 gate rows with their 8 up rows, the result is silu(x gate^T) * (x up^T)."""
    g = torch.Generator().manual_seed(18)
    A = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(2 * I, K, generator=g) * (2.0 / K ** 0.5)).bfloat16()
    Wp = ops.pack_weight(dev(W), gated=True)
    out = torch.full((M, I), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.gemv_mfma(dev(A), Wp, out, K, gated=True)
    gate, up = A.double() @ W[:I].double().T, A.double() @ W[I:].double().T
    want = torch.nn.functional.silu(gate) * up
    close(out, want, EPS["bfloat16"] * 1.5)
    # gate and up swapped, or pairs shifted, would show
    assert float((torch.nn.functional.silu(up) * gate - want).abs().max() / want.abs().max()) > 0.1


@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("M,N,K,columns", [(64, 128, 64, 64), (33, 200, 136, 32), (17, 72, 1000, 64), (32, 100, 264, 64), (20, 264, 520, 32),
                                           (50, 96, 4104, 64), (1, 40, 72, 32), (48, 3072, 2048, 32), (64, 1000, 3080, 64),
                                           (65, 72, 136, 32), (130, 200, 264, 64), (256, 96, 1000, 32), (200, 64, 2048, 64)])
def test_gemm_rows(ops, out_dtype, M, N, K, columns):
    """The product for 17 to 64 rows whose wavefronts each stream their own stages of K: both stagings of
    the rows (32 and 64), both widths of a block, tails in N, K and M, more and fewer stages than the
    rings hold; up to 256 rows as blocks of 64, the last one with 1, 2, 8 or all 64 rows."""
    g = torch.Generator().manual_seed(26)
    A = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(N, K, generator=g) * 0.1).bfloat16()
    W[N // 2, K - 8:] = 5.0   # one term that a wrong piece order or a lost tail cannot hide
    out = torch.full((M, N), 7.0, dtype=DT[out_dtype], device="cuda")
    ops.gemm_rows(dev(A), dev(W), out, columns=columns)
    want = A.double() @ W.double().T
    err = ((out.double().cpu() - want).abs() / (want.abs() + want.abs().mean())).max()
    assert float(err) <= (2e-5 if out_dtype == "float32" else 8e-3), f"error {float(err):.3g}"
    # rows of wider buffers, and an output with a row stride
    wide = torch.randn(M, K + 24, generator=g).bfloat16()
    wwide = (torch.randn(N, K + 16, generator=g) * 0.1).bfloat16()
    big = torch.zeros(M, N + 5, dtype=DT[out_dtype], device="cuda")
    ops.gemm_rows(dev(wide)[:, 8:K + 8], dev(wwide)[:, :K], big[:, :N], columns=columns)
    close(big[:, :N], wide[:, 8:K + 8].double() @ wwide[:, :K].double().T, EPS[out_dtype] * 3)
    assert bool((big[:, N:] == 0).all())


@pytest.mark.parametrize("M,N,K,groups,columns", [(64, 2048, 8192, 4, 32), (24, 100, 8200, 8, 64), (40, 48, 3000, 2, 32), (33, 64, 14336, 4, 64),
                                                  (17, 200, 1096, 3, 32), (100, 100, 2048, 2, 32), (192, 64, 3000, 3, 64)])
def test_gemm_rows_partial_products_sum_to_the_product(ops, M, N, K, groups, columns):
    g = torch.Generator().manual_seed(27)
    A = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    planes = torch.full((groups, M, N), 7.0, dtype=torch.float32, device="cuda")
    ops.gemm_rows(dev(A), dev(W), planes, columns=columns)
    close(planes.double().sum(0), A.double() @ W.double().T, 1e-5)
    per = ((K + groups - 1) // groups + 63) // 64 * 64          # a group's span: K / groups rounded up to whole stages of 64
    close(planes[0], A[:, :per].double() @ W[:, :per].double().T, 1e-5)
    close(planes[groups - 1], A[:, (groups - 1) * per:].double() @ W[:, (groups - 1) * per:].double().T, 1e-5)


@pytest.mark.parametrize("M,I,K", [(64, 1000, 2048), (20, 176, 1544), (37, 384, 144), (50, 8, 520), (32, 176, 4096), (33, 100, 3080),
                                   (70, 176, 520), (256, 100, 264)])
def test_gemm_rows_gated(ops, M, I, K):
    """The SwiGLU gating where the partial tiles of a block meet: w is [gate rows; up rows] as the checkpoint
    has them, a block takes 32 gate columns and the matching up columns."""
    g = torch.Generator().manual_seed(28)
    A = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(2 * I, K, generator=g) * (2.0 / K ** 0.5)).bfloat16()
    out = torch.full((M, I), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.gemm_rows(dev(A), dev(W), out, gated=True)
    gate, up = A.double() @ W[:I].double().T, A.double() @ W[I:].double().T
    want = torch.nn.functional.silu(gate) * up
    close(out, want, EPS["bfloat16"] * 1.5)
    assert float((torch.nn.functional.silu(up) * gate - want).abs().max() / want.abs().max()) > 0.1


def test_gemm_rows_refuses_what_it_cannot_do(ops):
    from burn_lm_amd.csrc.ops import KernelError
    a, w = dev(torch.zeros(257, 64).bfloat16()), dev(torch.zeros(8, 64).bfloat16())
    with pytest.raises(KernelError, match="M <= 256"):
        ops.gemm_rows(a, w, torch.zeros(257, 8, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(KernelError, match="32 without gating"):
        ops.gemm_rows(a[:8], w, torch.zeros(8, 4, dtype=torch.bfloat16, device="cuda"), gated=True, columns=32)
    with pytest.raises(KernelError, match="32 without gating"):
        ops.gemm_rows(a[:8], w, torch.zeros(8, 8, dtype=torch.bfloat16, device="cuda"), columns=48)
    with pytest.raises(KernelError, match="float32"):
        ops.gemm_rows(a[:8], w, torch.zeros(2, 8, 8, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(KernelError, match="do not fit"):
        ops.gemm_rows(a[:8], w, torch.zeros(8, 9, dtype=torch.bfloat16, device="cuda"))


def test_gemv_mfma_refuses_what_it_cannot_do(ops):
    from burn_lm_amd.csrc.ops import KernelError
    assert not ops.gemv_mfma_supported(65, 64, 64) and not ops.gemv_mfma_supported(4, 64, 60)
    assert not ops.gemv_mfma_supported(4, 64, 16392)
    # more rows leave fewer registers for each k-step: the K of one group shrinks
    assert ops.gemv_mfma_supported(32, 64, 4096) and not ops.gemv_mfma_supported(33, 64, 4096)
    assert ops.gemv_mfma_supported(64, 64, 2048) and not ops.gemv_mfma_supported(17, 64, 4104)
    assert [ops.gemv_mfma_group_limit(m) for m in (0, 1, 16, 17, 32, 33, 64, 65)] == [0, 16384, 16384, 4096, 4096, 2048, 2048, 0]
    wp = ops.pack_weight(dev(torch.zeros(8, 64).bfloat16()))
    with pytest.raises(KernelError, match="1..64"):
        ops.gemv_mfma(dev(torch.zeros(65, 64).bfloat16()), wp, torch.zeros(65, 8, dtype=torch.bfloat16, device="cuda"), 64)
    wide = ops.pack_weight(dev(torch.zeros(8, 4096).bfloat16()))
    with pytest.raises(KernelError, match="at most K=2048 per group"):
        ops.gemv_mfma(dev(torch.zeros(40, 4096).bfloat16()), wide, torch.zeros(40, 8, dtype=torch.bfloat16, device="cuda"), 4096)
    with pytest.raises(KernelError, match="packed weights"):
        ops.gemv_mfma(dev(torch.zeros(4, 64).bfloat16()), wp, torch.zeros(4, 40, dtype=torch.bfloat16, device="cuda"), 64)


@pytest.mark.parametrize("tile", [(128, 128), (256, 128), (256, 256), (128, 128, 4), (128, 64, 6)])
@pytest.mark.parametrize("M,N,K,groups,out_dtype", [(200, 136, 72, 1, "float32"), (300, 264, 200, 1, "bfloat16"),
                                                    (513, 520, 1096, 2, "float32"), (65, 31, 8, 1, "bfloat16"),
                                                    (129, 1000, 2048, 1, "bfloat16"), (260, 100, 4104, 4, "float32")])
def test_gemm_mfma(ops, tile, M, N, K, groups, out_dtype):
    """Matrix-core product for many rows: every tile shape; tails in M, N and K (a last stage that is
    no whole one, fewer stages than the ring holds), K cut into groups whose planes the reader sums,
    an output with a row stride and rows of a wider buffer."""
    g = torch.Generator().manual_seed(21)
    wide = torch.randn(M, K + 16, generator=g).bfloat16()
    W = torch.randn(N, K, generator=g).bfloat16()
    W[N // 2, K - 8:] = 40.0      # one term dominates a column: a wrong operand layout cannot hide in the noise
    A = wide[:, 8:K + 8]
    want = A.double() @ W.double().T
    if groups > 1:
        out = torch.full((groups, M, N), 7.0, dtype=torch.float32, device="cuda")
        ops.gemm_mfma(dev(wide)[:, 8:K + 8], dev(W), out, tile=tile)
        got = out.double().sum(0).cpu()
    else:
        big = torch.zeros(M, N + 8, dtype=DT[out_dtype], device="cuda")
        ops.gemm_mfma(dev(wide)[:, 8:K + 8], dev(W), big[:, :N], tile=tile)
        assert bool((big[:, N:] == 0).all())
        got = big[:, :N].double().cpu()
    err = ((got - want).abs() / (want.abs() + want.abs().mean())).max()
    assert float(err) <= (2e-5 if out_dtype == "float32" else 8e-3), f"error {float(err):.3g}"


@pytest.mark.parametrize("tile", [(128, 128), (256, 128), (256, 256), (128, 128, 4), (128, 64, 6)])
@pytest.mark.parametrize("M,I,K", [(70, 176, 64), (300, 264, 200), (257, 1000, 2048), (128, 8, 520)])
def test_gemm_mfma_gated(ops, tile, M, I, K):
    """The SwiGLU gating in the epilogue: a block takes gate columns and the matching up columns of
    the matrix as the checkpoint stores it ([gate rows; up rows])."""
    g = torch.Generator().manual_seed(22)
    A = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(2 * I, K, generator=g) * (2.0 / K ** 0.5)).bfloat16()
    out = torch.full((M, I), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.gemm_mfma(dev(A), dev(W), out, gated=True, tile=tile)
    gate, up = A.double() @ W[:I].double().T, A.double() @ W[I:].double().T
    want = torch.nn.functional.silu(gate) * up
    close(out, want, EPS["bfloat16"] * 1.5)
    assert float((torch.nn.functional.silu(up) * gate - want).abs().max() / want.abs().max()) > 0.1


def test_gemm_mfma_refuses_what_it_cannot_do(ops):
    from burn_lm_amd.csrc.ops import KernelError
    a, w = dev(torch.zeros(80, 64).bfloat16()), dev(torch.zeros(48, 64).bfloat16())
    with pytest.raises(KernelError, match="tile"):
        ops.gemm_mfma(a, w, torch.zeros(80, 48, dtype=torch.bfloat16, device="cuda"), tile=(64, 64))
    with pytest.raises(KernelError, match="do not fit"):
        ops.gemm_mfma(a, w, torch.zeros(80, 40, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(KernelError, match="bfloat16"):
        ops.gemm_mfma(a.float(), w, torch.zeros(80, 48, dtype=torch.float32, device="cuda"))
    with pytest.raises(KernelError, match="float32"):
        ops.gemm_mfma(a, w, torch.zeros(2, 80, 48, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(KernelError, match="K a multiple of 8"):
        ops.gemm_mfma(a[:, :60], w[:, :60], torch.zeros(80, 48, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(KernelError, match="one K group"):
        ops.gemm_mfma(a, w, torch.zeros(2, 80, 24, dtype=torch.float32, device="cuda"), gated=True)


def test_argmax_first_maximum_wins(ops):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(6, 1000, generator=g)
    x[1, 17] = x[1, 900] = 50.0
    x[2, 999] = 60.0
    x[3, 0] = 60.0
    x[4] = 0.0
    wide = torch.randn(6, 1200, generator=g)
    wide[:, :1000] = x
    wide[:, 1000:] = 100.0                       # beyond the vocabulary: must not be looked at
    got = ops.argmax(dev(wide)[:, :1000]).cpu().tolist()
    assert got == [int(x[0].argmax()), 17, 999, 0, 0, int(x[5].argmax())]


def test_sample_follows_the_temperature_distribution(ops):
    g = torch.Generator().manual_seed(8)
    V, R, T = 37, 40000, 0.7
    logits = torch.randn(V, generator=g) * 2
    probs = torch.softmax(logits.double() / T, 0)
    u = torch.rand(R, generator=g)
    got = ops.sample(dev(logits.expand(R, V).contiguous()), dev(u), T, 1.0).cpu()
    counts = torch.bincount(got.long(), minlength=V).double()
    chi2 = float(((counts - R * probs) ** 2 / (R * probs)).sum())
    assert chi2 < 80, f"chi-square {chi2:.1f} with 36 degrees of freedom"
    # inverse CDF in index order: the same u gives the same token, and u = 0 gives the first token with mass
    cdf = torch.cumsum(probs, 0)
    want = torch.searchsorted(cdf, u.double().clamp(max=float(cdf[-1]) - 1e-12), right=True)
    assert float((want == got).double().mean()) > 0.999
    # very low temperature is argmax
    cold = ops.sample(dev(logits.expand(50, V).contiguous()), dev(u[:50]), 1e-3, 1.0).cpu()
    assert bool((cold == int(logits.argmax())).all())


def test_sample_top_p_keeps_the_nucleus_only(ops):
    import plain_llama as P
    g = torch.Generator().manual_seed(9)
    V, R, T, p = 200, 20000, 1.3, 0.6
    logits = torch.randn(V, generator=g) * 1.5
    probs = P.temperature_softmax(logits.numpy(), T)
    kept = P.top_p_keep(probs, p)                 # crates/burn-lm-llama/src/generation/sampling.rs:50-63
    u = torch.rand(R, generator=g)
    got = ops.sample(dev(logits.expand(R, V).contiguous()), dev(u), T, p).cpu()
    seen = set(got.tolist())
    assert seen <= set(kept), f"tokens outside the nucleus were drawn: {sorted(seen - set(kept))}"
    assert seen == set(kept) or len(kept) - len(seen) <= 1
    sub = torch.tensor([probs[i] for i in kept]).double()
    sub = sub / sub.sum()
    counts = torch.tensor([(got == i).sum() for i in kept]).double()
    chi2 = float(((counts - R * sub) ** 2 / (R * sub)).sum())
    assert chi2 < 3 * len(kept) + 30
    # rows are independent: different logits per row, large vocabulary that is no power of two
    big = torch.randn(5, 50257, generator=g)
    big[3, 40000] = 30.0
    out = ops.sample(dev(big), dev(torch.full((5,), 0.5)), 0.8, 0.9).cpu()
    assert int(out[3]) == 40000 and all(0 <= int(t) < 50257 for t in out)


@pytest.mark.parametrize("V,ld", [(128256, 128256), (32003, 32003), (50257, 50260)])
def test_sample_large_vocabulary_matches_the_ordered_nucleus(ops, V, ld):
    """Vocabularies of real size (a multiple of four, an odd one that takes the scalar loads, a padded
    row stride): every draw lies in the plain implementation's nucleus and is the token at which the
    cumulative mass of the kept tokens, in index order, passes u; the same inputs give the same draws."""
    import plain_llama as P
    g = torch.Generator().manual_seed(41)
    R, T, p = 512, 0.8, 0.9
    logits = torch.randn(V, generator=g) * 2.5
    probs = P.temperature_softmax(logits.double().numpy(), T)
    kept = np.array(sorted(P.top_p_keep(probs, p)))
    cdf = np.cumsum(probs[kept]) / probs[kept].sum()
    u = torch.rand(R, generator=g)
    wide = torch.full((R, ld), 1e9)              # beyond the vocabulary: must not be looked at
    wide[:, :V] = logits
    x = dev(wide)[:, :V]
    got = ops.sample(x, dev(u), T, p).cpu().numpy()
    assert set(got.tolist()) <= set(kept.tolist()), "a token outside the nucleus was drawn"
    want = kept[np.minimum(np.searchsorted(cdf, u.double().numpy(), side="right"), len(kept) - 1)]
    assert (want == got).mean() > 0.99, f"{(want != got).sum()} of {R} draws differ from the ordered inverse CDF"
    again = ops.sample(x, dev(u), T, p).cpu().numpy()
    assert (again == got).all()
    # one or two rows are cut into more slices, and the uniforms may lie in pinned host memory: the same draws
    for rows in (1, 2, 3):
        few = ops.sample(x[:rows], u[:rows].clone().pin_memory(), T, p).cpu().numpy()
        assert (few == got[:rows]).all()
    # p = 1 keeps everything
    full = ops.sample(x, dev(u), T, 1.0).cpu().numpy()
    cdf1 = np.cumsum(probs)
    want1 = np.minimum(np.searchsorted(cdf1, u.double().numpy() * cdf1[-1], side="right"), V - 1)
    assert (want1 == full).mean() > 0.98


@pytest.mark.parametrize("pairing", ["interleaved", "half"])
@pytest.mark.parametrize("M,K,nh,nkv,hd", [(8, 2048, 4, 2, 64), (5, 264, 3, 1, 32), (16, 3072, 2, 2, 128), (1, 64, 6, 3, 64),
                                           (4, 4096, 2, 1, 64), (9, 3608, 3, 1, 32), (7, 2056, 2, 2, 32),
                                           (6, 520, 3, 1, 48), (16, 2048, 2, 1, 80), (8, 264, 30, 2, 128),
                                           (33, 2048, 4, 2, 64), (64, 520, 3, 1, 48), (20, 4096, 2, 1, 64), (17, 264, 30, 2, 128),
                                           (48, 2056, 2, 1, 32)])
def test_gemv_qkv_rope(ops, pairing, M, K, nh, nkv, hd):
    """The fused decode projection: equals the product, the rotation of its float result and the
    cache write done one after the other (in float64), for both pairings, with a padding row and
    scrambled pages; nothing else in the cache is touched."""
    from burn_lm_amd.parts.rope import PAIRING
    # adjacent pairs sit in one 16-column tile: any head size in steps of 16; pairs half a head apart
    # need two whole tiles per half: steps of 32
    # and from 17 rows on only adjacent pairs, with K up to 4096 for 32 rows and up to 2048 beyond
    takes = (pairing == "interleaved" or hd % 32 == 0) if M <= 16 else (pairing == "interleaved" and K <= (4096 if M <= 32 else 2048))
    assert ops.gemv_qkv_rope_supported(M, K, hd, PAIRING[pairing]) == takes
    if not takes:
        return

    def run(x, W, out, positions, token_seq, perm, cs, kd, vd, page, write_kv):
        ops.gemv_qkv_rope(x, ops.pack_weight(W), out, positions, token_seq, perm, cs, kd, vd, page, nh, nkv, hd, PAIRING[pairing],
                          write_kv=write_kv)

    _check_qkv_rope(run, pairing, M, K, nh, nkv, hd)


@pytest.mark.parametrize("M,K,nh,nkv,hd", [(33, 2048, 4, 2, 64), (64, 520, 3, 1, 48), (20, 4096, 2, 1, 64), (17, 264, 30, 2, 128),
                                           (48, 2056, 2, 1, 32), (64, 3072, 3, 1, 128), (40, 4104, 2, 2, 80), (32, 72, 1, 1, 6),
                                           (65, 264, 3, 1, 48), (128, 2048, 4, 2, 64), (200, 520, 2, 1, 128), (256, 72, 1, 1, 6)])
@pytest.mark.parametrize("columns,rows", [(32, 64), (64, 64), (32, 32)])
def test_gemm_rows_qkv_rope(ops, M, K, nh, nkv, hd, columns, rows):
    """The same for 17 to 256 rows on the product whose wavefronts stream their own stages of K: any K,
    head sizes that put two heads into a block's 32 or 64 columns or a head across several blocks, one to
    eight blocks of 64 or 32 rows (each with its own rows' positions and sequences)."""

    def run(x, W, out, positions, token_seq, perm, cs, kd, vd, page, write_kv):
        ops.gemm_rows_qkv_rope(x, W, out, positions, token_seq, perm, cs, kd, vd, page, nh, nkv, hd, write_kv=write_kv,
                               columns=columns, rows=rows)

    _check_qkv_rope(run, "interleaved", M, K, nh, nkv, hd)


def _check_qkv_rope(run, pairing, M, K, nh, nkv, hd):
    from burn_lm_amd.parts.rope import rope_frequencies
    g = torch.Generator().manual_seed(19)
    page, n_pages = 64, (16 if M <= 16 else max(64, M))       # four pages for every sequence
    N = (nh + 2 * nkv) * hd
    x = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(N, K, generator=g) / K ** 0.5).bfloat16()
    positions = torch.tensor([(37 * i + 5) % 250 for i in range(M)], dtype=torch.int32)
    token_seq = torch.arange(M, dtype=torch.int32)
    if M > 2:
        token_seq[2] = -1                      # a padding row: no cache write
        token_seq[3:] -= 1
    n_seq = int(token_seq.max()) + 1
    perm = torch.randperm(n_pages * 4, generator=g)[: n_seq * 4].reshape(n_seq, 4).to(torch.int32)
    freqs = torch.from_numpy(rope_frequencies(hd, 500000.0, (8, 1, 4, 32)))
    ang = torch.arange(256).double()[:, None] * freqs[None, :]
    cs = torch.stack([ang.cos(), ang.sin()], -1).float()
    k = torch.full((n_pages * 4, nkv, page, hd), 99.0).bfloat16()
    v = torch.full((n_pages * 4, nkv, hd, page), 99.0).bfloat16()
    kd, vd = dev(k), dev(v)
    out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    run(dev(x), dev(W), out, dev(positions), dev(token_seq), dev(perm), dev(cs), kd, vd, page, True)
    qkv = x.double() @ W.double().T
    q_ref = _rope_ref(qkv[:, : nh * hd].reshape(M, nh, hd), positions, freqs, pairing)
    k_ref = _rope_ref(qkv[:, nh * hd: (nh + nkv) * hd].reshape(M, nkv, hd), positions, freqs, pairing)
    v_ref = qkv[:, (nh + nkv) * hd:].reshape(M, nkv, hd)
    close(out[:, : nh * hd].reshape(M, nh, hd), q_ref, EPS["bfloat16"] * 1.5)
    assert bool((out[:, nh * hd:] == 7).all()), "only the queries are written to the buffer"
    kc, vc = kd.cpu().double(), vd.cpu().double()
    written = torch.zeros(n_pages * 4, page, dtype=torch.bool)
    for t in range(M):
        b = int(token_seq[t])
        if b < 0:
            continue
        p = int(positions[t]); pg = int(perm[b, p // page])
        written[pg, p % page] = True
        close(kc[pg, :, p % page], k_ref[t], EPS["bfloat16"] * 1.5)
        close(vc[pg, :, :, p % page], v_ref[t], EPS["bfloat16"] * 1.5)
    untouched = ~written[:, None, :, None].expand(n_pages * 4, nkv, page, hd)
    assert bool((kc[untouched] == 99).all()) and bool((vc.transpose(2, 3)[untouched] == 99).all())
    # a place that reads another's cache: queries only
    kd2 = dev(k)
    out2 = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    run(dev(x), dev(W), out2, dev(positions), dev(token_seq), dev(perm), dev(cs), kd2, dev(v), page, False)
    assert torch.equal(out2.cpu(), out.cpu()) and bool((kd2.cpu() == 99).all())
