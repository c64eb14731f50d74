"""A mixer with state of its own, and the architecture that uses it, are defined here, in the
test: registered, built from a model folder through the registry, and stepped, without a change
to the framework's files.  The toy is no model of anyone's: layer 0 is the framework's attention,
layer 1 a running decayed sum ``s_t = a * s_{t-1} + x_t W`` kept as fixed-size state per sequence,
and the order runs layer 0 twice, the second time reading the first run's keys and values."""
import json
import math
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu

TOY = dict(architectures=["ToyDecayLM"], width=48, inner=80, heads=4, kv_heads=2, head_dim=12, vocab=97,
           eps=1e-5, theta=10000.0, decay=0.8, max_positions=256)


def register_toy():
    from burn_lm_amd import registry
    from burn_lm_amd.models.plan import LayerPlan, ModelPlan, Place
    from burn_lm_amd.parts.base import Mixer, PartSpec, StateNeed, TensorSpec

    class DecayMixer(Mixer):
        """params: width, decay.  names: w.  State: one float32 vector per sequence."""

        def tensor_specs(self):
            return {self.names["w"]: TensorSpec((self.params["width"],) * 2)}

        def cache_need(self):
            return StateNeed((self.params["width"],), torch.float32)

        def bind(self, tensors, rt):
            self.rt, self.w, self.a = rt, tensors[self.names["w"]], float(self.params["decay"])

        def forward(self, x, step, view):
            u = self.rt.linear(x, self.w).float()
            out = torch.empty_like(u)
            row = 0
            for slot, n in zip(step.host_slots, step.host_new):   # tokens of a sequence run in order
                s = view.tensor[slot]
                for t in range(row, row + n):
                    s = self.a * s + u[t]
                    out[t] = s
                view.tensor[slot] = s
                row += n
            return out.to(self.rt.dtype)

    @dataclass(frozen=True)
    class ToyConfig:
        d: dict

        def __getattr__(self, k):
            return self.d[k]

    def plan(cfg, names=None):
        D = cfg.width
        norm = lambda n: PartSpec("rmsnorm", dict(width=D, eps=cfg.eps), dict(weight=n))
        ffn = lambda i: PartSpec("swiglu", dict(width=D, inner=cfg.inner),
                                 dict(gate=f"l{i}.gate", up=f"l{i}.up", down=f"l{i}.down"))
        attn = PartSpec("attention", dict(width=D, heads=cfg.heads, kv_heads=cfg.kv_heads, head_dim=cfg.head_dim,
                                          scale=1 / math.sqrt(cfg.head_dim)),
                        dict(q="l0.q", k="l0.k", v="l0.v", o="l0.o"))
        layers = [LayerPlan("pre_norm", mixer=attn, feed_forward=ffn(0), mixer_norm=norm("l0.n1"), ffn_norm=norm("l0.n2"),
                            position="rope"),
                  LayerPlan("pre_norm", mixer=PartSpec("toy_decay", dict(width=D, decay=cfg.decay), dict(w="l1.w")),
                            feed_forward=ffn(1), mixer_norm=norm("l1.n1"), ffn_norm=norm("l1.n2"))]
        return ModelPlan(vocab_size=cfg.vocab, width=D, max_positions=cfg.max_positions,
                         embedding=PartSpec("table", dict(vocab=cfg.vocab, width=D), dict(weight="emb")),
                         layers=layers, order=[Place(0), Place(1), Place(0, reads_cache_of=0)],
                         final_norm=norm("norm"), head=PartSpec("linear", dict(vocab=cfg.vocab, width=D), dict(weight="emb")),
                         positions={"rope": PartSpec("rope", dict(head_dim=cfg.head_dim, theta=cfg.theta,
                                                                  pairing="interleaved", scaling=None))})

    registry.register_part("mixer", "toy_decay", DecayMixer)
    registry.register_architecture(registry.Architecture("ToyDecayLM", read_config=lambda d: ToyConfig(d), plan=plan))


def toy_weights(seed=3):
    c = TOY
    g = torch.Generator().manual_seed(seed)
    m = lambda *s: (torch.randn(*s, generator=g) * 0.15).bfloat16()
    n = lambda: (1 + 0.1 * torch.randn(c["width"], generator=g)).bfloat16()
    D, I, hd = c["width"], c["inner"], c["head_dim"]
    t = {"emb": m(c["vocab"], D), "norm": n(), "l1.w": m(D, D),
         "l0.q": m(c["heads"] * hd, D), "l0.k": m(c["kv_heads"] * hd, D), "l0.v": m(c["kv_heads"] * hd, D),
         "l0.o": m(D, c["heads"] * hd)}
    for i in (0, 1):
        t.update({f"l{i}.gate": m(I, D), f"l{i}.up": m(I, D), f"l{i}.down": m(D, I), f"l{i}.n1": n(), f"l{i}.n2": n()})
    return t


def toy_plain(tokens, t):
    """The toy's whole-sequence forward in float64, from the plain parts."""
    c = TOY
    w = {k: v.double().numpy() for k, v in t.items()}
    freqs = P.rope_base_frequencies(c["head_dim"], c["theta"])
    ffn = lambda i, x: P.swiglu_feed_forward(x, w[f"l{i}.gate"], w[f"l{i}.up"], w[f"l{i}.down"])
    attn = lambda x: P.attention_layer(x, w["l0.q"], w["l0.k"], w["l0.v"], w["l0.o"], c["heads"], c["kv_heads"],
                                       c["head_dim"], freqs)
    h = w["emb"][np.asarray(tokens)][None]
    # place 0: attention layer
    x0 = P.rms_norm(h, w["l0.n1"], c["eps"])
    h = h + attn(x0)
    h = h + ffn(0, P.rms_norm(h, w["l0.n2"], c["eps"]))
    # place 1: decayed running sum
    u = P.rms_norm(h, w["l1.n1"], c["eps"]) @ w["l1.w"].T
    s, outs = np.zeros(c["width"]), []
    for i in range(u.shape[1]):
        s = c["decay"] * s + u[0, i]
        outs.append(s)
    h = h + np.stack(outs)[None]
    h = h + ffn(1, P.rms_norm(h, w["l1.n2"], c["eps"]))
    # place 2: layer 0 again, queries from the new stream, keys and values of place 0
    x2 = P.rms_norm(h, w["l0.n1"], c["eps"])
    b, T = 1, x2.shape[1]
    q = (x2 @ w["l0.q"].T).reshape(b, T, c["heads"], c["head_dim"]).swapaxes(1, 2)
    k = (x0 @ w["l0.k"].T).reshape(b, T, c["kv_heads"], c["head_dim"]).swapaxes(1, 2)
    v = (x0 @ w["l0.v"].T).reshape(b, T, c["kv_heads"], c["head_dim"]).swapaxes(1, 2)
    pos = np.arange(T)
    o = P.scaled_attention(P.rope_interleaved(q, pos, freqs), P.rope_interleaved(k, pos, freqs), v, P.hidden_mask(T, T))
    h = h + o.swapaxes(1, 2).reshape(b, T, -1) @ w["l0.o"].T
    h = h + ffn(0, P.rms_norm(h, w["l0.n2"], c["eps"]))
    return (P.rms_norm(h, w["norm"], c["eps"]) @ w["emb"].T)[0]


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype, tol):
    from burn_lm_amd.cache.cache import KVView, StateView
    from burn_lm_amd.engine.loading import load_engine
    from burn_lm_amd.weights import safetensors_io as st
    register_toy()
    t = toy_weights()
    json.dump(TOY, open(tmp_path / "config.json", "w"))
    st.write_file(str(tmp_path / "model.safetensors"), t.items())
    eng = load_engine(str(tmp_path), dtype=dtype, max_tokens=512, max_seqs=4)
    views = eng.cache.views
    assert isinstance(views[0], KVView) and isinstance(views[1], StateView) and isinstance(views[2], KVView)
    assert views[2].k.data_ptr() == views[0].k.data_ptr() and not views[2].store
    assert eng.cache.groups[0].k_storage.shape[0] == 1 and views[1].tensor.shape == (4, 48)
    rng = np.random.default_rng(0)
    reqs = [[int(x) for x in rng.integers(0, 97, n)] for n in (70, 9, 33)]
    want = [toy_plain(r, t) for r in reqs]
    err = lambda got, w: float(np.abs(got.double().cpu().numpy() - w).max() / np.abs(w).max())
    # whole, each alone
    for r, w in zip(reqs, want):
        s = eng.open()
        assert err(eng.step([(s, r, list(range(len(r))))]), w) <= tol
        eng.close(s)
    # unequal batch: prompts in one step, then one token each; the shortest ends first; state and
    # slots are used again by a second batch
    for _ in range(2):
        slots = [eng.open() for _ in reqs]
        cut = [len(r) - 8 for r in reqs]
        got = eng.step([(s, r[:c], list(range(c))) for s, r, c in zip(slots, reqs, cut)])
        o = 0
        for r, c, w in zip(reqs, cut, want):
            assert err(got[o:o + c], w[:c]) <= tol
            o += c
        for k in range(8):
            live = [i for i in range(3) if not (i == 1 and k >= 4)]
            got = eng.step([(slots[i], [reqs[i][cut[i] + k]], [0]) for i in live])
            for row, i in enumerate(live):
                assert err(got[row], want[i][cut[i] + k]) <= tol, f"request {i}, decode step {k}"
            if k == 3:
                eng.close(slots[1])
        eng.close(slots[0]); eng.close(slots[2])
    assert eng.cache.pages_in_use() == 0


def test_a_windowed_attention_layer_beside_a_full_one(tmp_path):
    """Two attention layers of one model with different needs: the first keeps a window of 40 keys
    (its group gives pages back as they fall out of the window), the second all keys.  Prompts longer
    than the window, then decoding across the window's edge and page edges, against the plain
    attention with the window's mask; the page pools of the two groups are checked as well."""
    import math as _m
    from burn_lm_amd import registry
    from burn_lm_amd.engine.loading import load_engine
    from burn_lm_amd.models.plan import LayerPlan, ModelPlan, Place
    from burn_lm_amd.parts.base import PartSpec
    from burn_lm_amd.weights import safetensors_io as st
    W = 40
    c = dict(architectures=["ToyWindowLM"], width=64, inner=96, heads=4, kv_heads=2, head_dim=16, vocab=101, eps=1e-5,
             theta=10000.0, max_positions=512)

    def plan(cfg, names=None):
        D = cfg["width"]
        norm = lambda n: PartSpec("rmsnorm", dict(width=D, eps=cfg["eps"]), dict(weight=n))
        layer = lambda i, window: LayerPlan(
            "pre_norm",
            mixer=PartSpec("attention", dict(width=D, heads=cfg["heads"], kv_heads=cfg["kv_heads"], head_dim=cfg["head_dim"],
                                             scale=1 / _m.sqrt(cfg["head_dim"]), window=window),
                           dict(q=f"l{i}.q", k=f"l{i}.k", v=f"l{i}.v", o=f"l{i}.o")),
            feed_forward=PartSpec("swiglu", dict(width=D, inner=cfg["inner"]),
                                  dict(gate=f"l{i}.gate", up=f"l{i}.up", down=f"l{i}.down")),
            mixer_norm=norm(f"l{i}.n1"), ffn_norm=norm(f"l{i}.n2"), position="rope")
        return ModelPlan(vocab_size=cfg["vocab"], width=D, max_positions=cfg["max_positions"],
                         embedding=PartSpec("table", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")),
                         layers=[layer(0, W), layer(1, 0)], order=[Place(0), Place(1)], final_norm=norm("norm"),
                         head=PartSpec("linear", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")),
                         positions={"rope": PartSpec("rope", dict(head_dim=cfg["head_dim"], theta=cfg["theta"],
                                                                  pairing="interleaved", scaling=None))})

    registry.register_architecture(registry.Architecture("ToyWindowLM", read_config=lambda d: d, plan=plan))
    g = torch.Generator().manual_seed(21)
    m = lambda *s: (torch.randn(*s, generator=g) * 0.2).bfloat16()
    n = lambda: (1 + 0.1 * torch.randn(c["width"], generator=g)).bfloat16()
    D, I, hd = c["width"], c["inner"], c["head_dim"]
    t = {"emb": m(c["vocab"], D), "norm": n()}
    for i in (0, 1):
        t.update({f"l{i}.q": m(c["heads"] * hd, D), f"l{i}.k": m(c["kv_heads"] * hd, D), f"l{i}.v": m(c["kv_heads"] * hd, D),
                  f"l{i}.o": m(D, c["heads"] * hd), f"l{i}.gate": m(I, D), f"l{i}.up": m(I, D), f"l{i}.down": m(D, I),
                  f"l{i}.n1": n(), f"l{i}.n2": n()})
    json.dump(c, open(tmp_path / "config.json", "w"))
    st.write_file(str(tmp_path / "model.safetensors"), t.items())
    w = {k: v.double().numpy() for k, v in t.items()}
    freqs = P.rope_base_frequencies(hd, c["theta"])

    def plain(tokens):
        T = len(tokens)
        h = w["emb"][np.asarray(tokens)][None]
        pos = np.arange(T)
        for i, window in ((0, W), (1, 0)):
            x = P.rms_norm(h, w[f"l{i}.n1"], c["eps"])
            q = (x @ w[f"l{i}.q"].T).reshape(1, T, c["heads"], hd).swapaxes(1, 2)
            k = (x @ w[f"l{i}.k"].T).reshape(1, T, c["kv_heads"], hd).swapaxes(1, 2)
            v = (x @ w[f"l{i}.v"].T).reshape(1, T, c["kv_heads"], hd).swapaxes(1, 2)
            hidden = P.hidden_mask(T, T) if T > 1 else np.zeros((1, 1), dtype=bool)
            if window:
                hidden = hidden | (pos[:, None] - pos[None, :] >= window)   # key j is seen iff p - j < window
            o = P.scaled_attention(P.rope_interleaved(q, pos, freqs), P.rope_interleaved(k, pos, freqs), v, hidden)
            h = h + o.swapaxes(1, 2).reshape(1, T, -1) @ w[f"l{i}.o"].T
            h = h + P.swiglu_feed_forward(P.rms_norm(h, w[f"l{i}.n2"], c["eps"]), w[f"l{i}.gate"], w[f"l{i}.up"], w[f"l{i}.down"])
        return (P.rms_norm(h, w["norm"], c["eps"]) @ w["emb"].T)[0]

    rng = np.random.default_rng(5)
    reqs = [[int(x) for x in rng.integers(0, 101, L)] for L in (150, 30, 75)]
    want = [plain(r) for r in reqs]
    err = lambda got, ww: float(np.abs(got.double().cpu().numpy() - ww).max() / np.abs(ww).max())
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 3e-2)):
        eng = load_engine(str(tmp_path), dtype=dtype, max_tokens=1024, max_seqs=4)
        assert len(eng.cache.groups) == 2 and {g_.need.window for g_ in eng.cache.groups} == {0, W}
        slots = [eng.open() for _ in reqs]
        cut = [len(r) - 20 for r in reqs]
        got = eng.step([(s, r[:k], list(range(k))) for s, r, k in zip(slots, reqs, cut)])
        o = 0
        for r, k, ww in zip(reqs, cut, want):
            assert err(got[o:o + k], ww[:k]) <= tol, f"{dtype} prompt"
            o += k
        for j in range(20):
            got = eng.step([(s, [r[k + j]], [0]) for s, r, k in zip(slots, reqs, cut)])
            for i in range(3):
                assert err(got[i], want[i][cut[i] + j]) <= tol, f"{dtype} request {i} decode {j}"
        win = next(g_ for g_ in eng.cache.groups if g_.need.window == W)
        full = next(g_ for g_ in eng.cache.groups if g_.need.window == 0)
        # request 0 holds 150 tokens: 3 pages in the full group; in the windowed group only the pages
        # that still hold keys 111.. (pages 1 and 2), page 0 went back to the pool
        assert [p >= 0 for p in win.tables[slots[0]]] == [False, True, True]
        assert all(p >= 0 for p in full.tables[slots[0]]) and len(full.tables[slots[0]]) == 3
        for s in slots:
            eng.close(s)
        assert eng.cache.pages_in_use() == 0


def test_a_mixer_whose_values_have_a_size_and_a_head_count_of_their_own(tmp_path):
    """The cache keeps keys and values apart, so a mixer may ask for values of another head size and
    another head count than its keys.  The toy, defined here and written in torch: 4 query heads over
    2 key heads of size 8, and one value head of size 20 that all query heads share; no rotation.  It
    writes and reads its pages through the page table by itself."""
    from burn_lm_amd import registry
    from burn_lm_amd.engine.loading import load_engine
    from burn_lm_amd.models.plan import LayerPlan, ModelPlan, Place
    from burn_lm_amd.parts.base import KVNeed, Mixer, PartSpec, TensorSpec
    from burn_lm_amd.weights import safetensors_io as st
    c = dict(architectures=["ToyWideValueLM"], width=40, inner=56, heads=4, kv_heads=2, key_dim=8, value_dim=20, vocab=89,
             eps=1e-5, max_positions=512)
    H, G, kd, vd, D = c["heads"], c["kv_heads"], c["key_dim"], c["value_dim"], c["width"]

    class WideValueMixer(Mixer):
        def tensor_specs(self):
            n = self.names
            return {n["q"]: TensorSpec((H * kd, D)), n["k"]: TensorSpec((G * kd, D)), n["v"]: TensorSpec((vd, D)),
                    n["o"]: TensorSpec((D, H * vd))}

        def cache_need(self):
            return KVNeed(G, kd, value_dim=vd, n_value_heads=1)

        def bind(self, tensors, rt):
            self.rt = rt
            self.q, self.k, self.v, self.o = (tensors[self.names[x]] for x in "qkvo")

        def forward(self, x, step, view):
            T = x.shape[0]
            q = self.rt.linear(x, self.q).float().view(T, H, kd)
            k = self.rt.linear(x, self.k).view(T, G, kd)
            v = self.rt.linear(x, self.v).view(T, vd)
            table, pos, page = view.block_table(step).cpu(), step.positions.cpu().tolist(), view.page_size
            out = torch.zeros(T, H, vd, device=x.device)
            row = 0
            for b, n in enumerate(step.host_new):
                for t in range(row, row + n):
                    p = int(table[b, pos[t] // page])
                    view.k[p, :, pos[t] % page] = k[t]
                    view.v[p, 0, :, pos[t] % page] = v[t]
                L = pos[row + n - 1] + 1
                pages = table[b, :(L + page - 1) // page].long().to(x.device)
                keys = view.k[pages].permute(1, 0, 2, 3).reshape(G, -1, kd)[:, :L].float()       # [G, L, kd]
                values = view.v[pages][:, 0].permute(1, 0, 2).reshape(vd, -1)[:, :L].float()     # [vd, L]
                for t in range(row, row + n):
                    s = torch.einsum("hd,hld->hl", q[t], keys.repeat_interleave(H // G, 0)[:, :pos[t] + 1]) / math.sqrt(kd)
                    out[t] = torch.softmax(s, -1) @ values[:, :pos[t] + 1].T
                row += n
            return self.rt.linear(out.view(T, H * vd).to(self.rt.dtype), self.o)

    def plan(cfg, names=None):
        norm = lambda n: PartSpec("rmsnorm", dict(width=D, eps=cfg["eps"]), dict(weight=n))
        layer = LayerPlan("pre_norm", mixer=PartSpec("toy_wide_value", {}, dict(q="q", k="k", v="v", o="o")),
                          feed_forward=PartSpec("swiglu", dict(width=D, inner=cfg["inner"]), dict(gate="gate", up="up", down="down")),
                          mixer_norm=norm("n1"), ffn_norm=norm("n2"))
        return ModelPlan(vocab_size=cfg["vocab"], width=D, max_positions=cfg["max_positions"],
                         embedding=PartSpec("table", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")),
                         layers=[layer], order=[Place(0)], final_norm=norm("norm"),
                         head=PartSpec("linear", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")), positions={})

    registry.register_part("mixer", "toy_wide_value", WideValueMixer)
    registry.register_architecture(registry.Architecture("ToyWideValueLM", read_config=lambda d: d, plan=plan))
    g = torch.Generator().manual_seed(8)
    m = lambda *s: (torch.randn(*s, generator=g) * 0.2).bfloat16()
    n = lambda: (1 + 0.1 * torch.randn(D, generator=g)).bfloat16()
    t = {"emb": m(c["vocab"], D), "norm": n(), "n1": n(), "n2": n(), "q": m(H * kd, D), "k": m(G * kd, D), "v": m(vd, D),
         "o": m(D, H * vd), "gate": m(c["inner"], D), "up": m(c["inner"], D), "down": m(D, c["inner"])}
    json.dump(c, open(tmp_path / "config.json", "w"))
    st.write_file(str(tmp_path / "model.safetensors"), t.items())
    w = {k: v.double().numpy() for k, v in t.items()}

    def plain(tokens):
        T = len(tokens)
        h = w["emb"][np.asarray(tokens)][None]
        x = P.rms_norm(h, w["n1"], c["eps"])
        q = (x @ w["q"].T).reshape(1, T, H, kd).swapaxes(1, 2)
        k = (x @ w["k"].T).reshape(1, T, G, kd).swapaxes(1, 2)
        v = np.repeat((x @ w["v"].T).reshape(1, T, 1, vd).swapaxes(1, 2), G, axis=1)      # the one value head, for every group
        o = P.scaled_attention(q, k, v, P.hidden_mask(T, T))
        h = h + o.swapaxes(1, 2).reshape(1, T, -1) @ w["o"].T
        h = h + P.swiglu_feed_forward(P.rms_norm(h, w["n2"], c["eps"]), w["gate"], w["up"], w["down"])
        return (P.rms_norm(h, w["norm"], c["eps"]) @ w["emb"].T)[0]

    rng = np.random.default_rng(6)
    reqs = [[int(x) for x in rng.integers(0, c["vocab"], L)] for L in (100, 17, 70)]
    want = [plain(r) for r in reqs]
    err = lambda got, ww: float(np.abs(got.double().cpu().numpy() - ww).max() / np.abs(ww).max())
    eng = load_engine(str(tmp_path), dtype="float32", max_tokens=512, max_seqs=3)
    group = eng.cache.groups[0]
    assert group.k_storage.shape[2:] == (G, 64 * kd) and group.v_storage.shape[2:] == (1, vd * 64)
    for _ in range(2):                       # twice, so that slots and pages are used again
        slots = [eng.open() for _ in reqs]
        cut = [len(r) - 6 for r in reqs]
        got = eng.step([(s, r[:k], list(range(k))) for s, r, k in zip(slots, reqs, cut)])
        o = 0
        for k, ww in zip(cut, want):
            assert err(got[o:o + k], ww[:k]) <= 2e-5
            o += k
        for j in range(6):
            got = eng.step([(s, [r[k + j]], [0]) for s, r, k in zip(slots, reqs, cut)])
            for i in range(3):
                assert err(got[i], want[i][cut[i] + j]) <= 2e-5, (i, j)
        for s in slots:
            eng.close(s)
    assert eng.cache.pages_in_use() == 0

