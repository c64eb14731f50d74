"""A feed-forward with routing and another position encoding, defined here in the test, chosen for
one layer of a two-layer toy while the other layer keeps the framework's own parts: registered,
built from a model folder and stepped without a change to the framework's files.  The toy is no
model of anyone's.

* ``toy_routed``: three small gated experts; a linear router picks one per token (float32 logits,
  highest wins) and its softmax probability weighs the expert's output.
* ``toy_key_fade``: no rotation; the key written at position p is scaled by 1 / (1 + p / 64),
  the query is left alone.
"""
import json
import math

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu

TOY = dict(architectures=["ToyRoutedLM"], width=80, inner=112, expert_inner=48, experts=3, heads=5, kv_heads=5,
           head_dim=16, vocab=131, eps=1e-6, theta=10000.0, max_positions=512)


def register_toy():
    from burn_lm_amd import registry
    from burn_lm_amd.models.plan import LayerPlan, ModelPlan, Place
    from burn_lm_amd.parts.base import FeedForward, PartSpec, PositionEncoding, TensorSpec

    class RoutedFeedForward(FeedForward):
        """params: width, inner, experts.  names: router, gate{e}, up{e}, down{e}."""

        def tensor_specs(self):
            D, I, E = self.params["width"], self.params["inner"], self.params["experts"]
            specs = {self.names["router"]: TensorSpec((E, D))}
            for e in range(E):
                specs[self.names[f"gate{e}"]] = TensorSpec((I, D))
                specs[self.names[f"up{e}"]] = TensorSpec((I, D))
                specs[self.names[f"down{e}"]] = TensorSpec((D, I))
            return specs

        def bind(self, tensors, rt):
            self.rt = rt
            self.router = tensors[self.names["router"]].float()
            E = self.params["experts"]
            self.w = [tuple(tensors[self.names[f"{r}{e}"]] for r in ("gate", "up", "down")) for e in range(E)]

        def forward(self, x, step):
            logits = x.float() @ self.router.T                      # router in float32
            prob, pick = torch.softmax(logits, -1).max(-1)
            out = torch.zeros(x.shape[0], self.params["width"], dtype=torch.float32, device=x.device)
            for e, (wg, wu, wd) in enumerate(self.w):
                idx = (pick == e).nonzero().squeeze(1)              # tokens of this expert
                if idx.numel() == 0:
                    continue
                xe = x[idx].contiguous()
                act = torch.nn.functional.silu(self.rt.linear(xe, wg).float()) * self.rt.linear(xe, wu).float()
                out[idx] = self.rt.linear(act.to(self.rt.dtype), wd).float() * prob[idx, None]
            return out.to(self.rt.dtype)

    class KeyFade(PositionEncoding):
        """params: fade.  Keys are scaled by 1 / (1 + position / fade) and stored; values stored as they are."""

        def encode_and_store(self, qkv, step, view, heads, kv_heads, head_dim, store=True):
            if not store:
                return
            T = qkv.shape[0]
            k = qkv[:, heads * head_dim:(heads + kv_heads) * head_dim].reshape(T, kv_heads, head_dim)
            v = qkv[:, (heads + kv_heads) * head_dim:].reshape(T, kv_heads, head_dim)
            pos = step.positions.long()
            live = step.token_seq >= 0
            seq = step.token_seq.clamp(min=0).long()
            pages = view.block_table(step)[seq, pos // view.page_size].long()
            live = live & (pages >= 0)
            pages, slots = pages[live], (pos % view.page_size)[live]
            fade = 1.0 / (1.0 + pos[live].float() / float(self.params["fade"]))
            view.k[pages, :, slots, :] = (k[live].float() * fade[:, None, None]).to(view.k.dtype)
            view.v[pages, :, :, slots] = v[live]

    def plan(cfg, names=None):
        D = cfg["width"]
        norm = lambda n: PartSpec("rmsnorm", dict(width=D, eps=cfg["eps"]), dict(weight=n))
        attn = lambda i: PartSpec("attention", dict(width=D, heads=cfg["heads"], kv_heads=cfg["kv_heads"],
                                                    head_dim=cfg["head_dim"], scale=1 / math.sqrt(cfg["head_dim"])),
                                  dict(q=f"l{i}.q", k=f"l{i}.k", v=f"l{i}.v", o=f"l{i}.o"))
        routed_names = dict(router="l1.router")
        for e in range(cfg["experts"]):
            routed_names.update({f"gate{e}": f"l1.e{e}.gate", f"up{e}": f"l1.e{e}.up", f"down{e}": f"l1.e{e}.down"})
        layers = [
            LayerPlan("pre_norm", mixer=attn(0),
                      feed_forward=PartSpec("swiglu", dict(width=D, inner=cfg["inner"]),
                                            dict(gate="l0.gate", up="l0.up", down="l0.down")),
                      mixer_norm=norm("l0.n1"), ffn_norm=norm("l0.n2"), position="rope"),
            LayerPlan("pre_norm", mixer=attn(1),
                      feed_forward=PartSpec("toy_routed", dict(width=D, inner=cfg["expert_inner"],
                                                               experts=cfg["experts"]), routed_names),
                      mixer_norm=norm("l1.n1"), ffn_norm=norm("l1.n2"), position="fade")]
        return ModelPlan(vocab_size=cfg["vocab"], width=D, max_positions=cfg["max_positions"],
                         embedding=PartSpec("table", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")),
                         layers=layers, order=[Place(0), Place(1)], final_norm=norm("norm"),
                         head=PartSpec("linear", dict(vocab=cfg["vocab"], width=D), dict(weight="head")),
                         positions={"rope": PartSpec("rope", dict(head_dim=cfg["head_dim"], theta=cfg["theta"],
                                                                  pairing="interleaved", scaling=None)),
                                    "fade": PartSpec("toy_key_fade", dict(fade=64.0))})

    registry.register_part("feed_forward", "toy_routed", RoutedFeedForward)
    registry.register_part("position", "toy_key_fade", KeyFade)
    registry.register_architecture(registry.Architecture("ToyRoutedLM", read_config=lambda d: d, plan=plan))


def toy_weights(seed=5):
    c = TOY
    g = torch.Generator().manual_seed(seed)
    m = lambda *s: (torch.randn(*s, generator=g) * 0.15).bfloat16()
    n = lambda: (1 + 0.1 * torch.randn(c["width"], generator=g)).bfloat16()
    D, I, J, hd = c["width"], c["inner"], c["expert_inner"], c["head_dim"]
    t = {"emb": m(c["vocab"], D), "head": m(c["vocab"], D), "norm": n(),
         "l0.gate": m(I, D), "l0.up": m(I, D), "l0.down": m(D, I),
         "l1.router": (torch.randn(c["experts"], D, generator=g) * 0.6).bfloat16()}
    for i in (0, 1):
        t.update({f"l{i}.q": m(c["heads"] * hd, D), f"l{i}.k": m(c["kv_heads"] * hd, D), f"l{i}.v": m(c["kv_heads"] * hd, D),
                  f"l{i}.o": m(D, c["heads"] * hd), f"l{i}.n1": n(), f"l{i}.n2": n()})
    for e in range(c["experts"]):
        t.update({f"l1.e{e}.gate": m(J, D), f"l1.e{e}.up": m(J, D), f"l1.e{e}.down": m(D, J)})
    return t


def toy_plain(tokens, t):
    """Whole-sequence forward in float64 from the plain parts; also the router's margin per token
    (the gap between its two highest logits)."""
    c = TOY
    w = {k: v.double().numpy() for k, v in t.items()}
    T, hd = len(tokens), c["head_dim"]
    pos = np.arange(T)
    freqs = P.rope_base_frequencies(hd, c["theta"])
    h = w["emb"][np.asarray(tokens)][None]
    # layer 0: the framework's parts
    h = h + P.attention_layer(P.rms_norm(h, w["l0.n1"], c["eps"]), w["l0.q"], w["l0.k"], w["l0.v"], w["l0.o"],
                              c["heads"], c["kv_heads"], hd, freqs)
    h = h + P.swiglu_feed_forward(P.rms_norm(h, w["l0.n2"], c["eps"]), w["l0.gate"], w["l0.up"], w["l0.down"])
    # layer 1: keys fade with their position, no rotation; routed experts
    x = P.rms_norm(h, w["l1.n1"], c["eps"])
    q = (x @ w["l1.q"].T).reshape(1, T, c["heads"], hd).swapaxes(1, 2)
    k = (x @ w["l1.k"].T).reshape(1, T, c["kv_heads"], hd).swapaxes(1, 2)
    v = (x @ w["l1.v"].T).reshape(1, T, c["kv_heads"], hd).swapaxes(1, 2)
    k = k / (1.0 + pos / 64.0)[None, None, :, None]
    hidden = P.hidden_mask(T, T) if T > 1 else np.zeros((1, 1), dtype=bool)
    o = P.scaled_attention(q, k, v, hidden)
    h = h + o.swapaxes(1, 2).reshape(1, T, -1) @ w["l1.o"].T
    x = P.rms_norm(h, w["l1.n2"], c["eps"])[0]
    logits = x @ w["l1.router"].T
    prob = P.softmax(logits, -1)
    pick = logits.argmax(-1)
    srt = np.sort(logits, -1)
    margin = srt[:, -1] - srt[:, -2]
    f = np.zeros_like(x)
    for i in range(T):
        e = int(pick[i])
        f[i] = P.swiglu_feed_forward(x[i][None], w[f"l1.e{e}.gate"], w[f"l1.e{e}.up"], w[f"l1.e{e}.down"])[0] * prob[i, e]
    h = h + f[None]
    return (P.rms_norm(h, w["norm"], c["eps"]) @ w["head"].T)[0], margin, pick


@pytest.mark.parametrize("dtype,tol,min_margin", [("float32", 2e-5, 1e-4), ("bfloat16", 3e-2, 0.15)])
def test_a_routed_feed_forward_and_another_position_encoding(tmp_path, dtype, tol, min_margin):
    from burn_lm_amd.engine.loading import load_engine
    from burn_lm_amd.weights import safetensors_io as st
    register_toy()
    t = toy_weights()
    json.dump(TOY, open(tmp_path / "config.json", "w"))
    st.write_file(str(tmp_path / "model.safetensors"), t.items())
    eng = load_engine(str(tmp_path), dtype=dtype, max_tokens=1024, max_seqs=4)
    kinds = [(type(b.mixer).__name__, type(b.feed_forward).__name__) for b in eng.model.blocks]
    assert kinds == [("Attention", "SwiGLU"), ("Attention", "RoutedFeedForward")], kinds
    assert not eng.graphs.enabled        # the toy parts do not declare themselves graph-safe

    rng = np.random.default_rng(2)
    reqs = [[int(x) for x in rng.integers(0, TOY["vocab"], L)] for L in (150, 9, 70)]
    plain = [toy_plain(r, t) for r in reqs]
    assert len({int(e) for _, _, pick in plain for e in pick}) == TOY["experts"], "every expert must get tokens"
    checked = total = 0

    def compare(got, req, p):
        nonlocal checked, total
        want, margin, _ = plain[req]
        total += 1
        if margin[p] < min_margin:      # the router's two best are too close for this precision to tell
            return
        checked += 1
        err = float(np.abs(got.double().cpu().numpy() - want[p]).max() / np.abs(want).max())
        assert err <= tol, f"{dtype} request {req} position {p}: {err:.3g}"

    slots = [eng.open() for _ in reqs]
    cut = [len(r) - 6 for r in reqs]
    got = eng.step([(s, r[:k], list(range(k))) for s, r, k in zip(slots, reqs, cut)])
    o = 0
    for i, k in enumerate(cut):
        for p in range(k):
            compare(got[o + p], i, p)
        o += k
    for j in range(6):                  # one token each, across the page edge of the long request
        got = eng.step([(s, [r[k + j]], [0]) for s, r, k in zip(slots, reqs, cut)])
        for i in range(3):
            compare(got[i], i, cut[i] + j)
    assert checked >= 0.8 * total, f"only {checked} of {total} positions were decisive enough to compare"
    for s in slots:
        eng.close(s)
    assert eng.cache.pages_in_use() == 0


def test_a_toy_encoding_with_a_fused_projection_asks_the_runtime_for_its_geometry(tmp_path):
    """A position encoding defined here that fuses the q/k/v projection with its own work (it turns
    nothing: a table of cosine one and sine zero, handed to the library's fused kernels as its own)
    holds no threshold: which launch geometry suits which number of rows is the runtime's answer
    (Runtime.qkv_plan), and the encoding only checks what its own kernels take.  Steps of 1 to 300 rows
    meet every answer (packed, row ring with 32 and 64 rows staged, none); the logits are the plain
    attention's without rotation."""
    from burn_lm_amd import registry
    from burn_lm_amd.engine.loading import load_engine
    from burn_lm_amd.models.plan import LayerPlan, ModelPlan, Place
    from burn_lm_amd.parts.base import PartSpec, PositionEncoding
    from burn_lm_amd.weights import safetensors_io as st
    asked = []

    class Still(PositionEncoding):
        graph_safe = True

        def prepare(self, n_positions, rt):
            hd = self.params["head_dim"]
            self.table = torch.stack([torch.ones(n_positions, hd // 2), torch.zeros(n_positions, hd // 2)], -1).to(rt.device)

        def encode_and_store(self, qkv, step, view, heads, kv_heads, head_dim, store=True):
            self.rt.ops.rope_kv_write(qkv, step.positions, step.token_seq, view.block_table(step), self.table, view.k, view.v,
                                      view.page_size, heads, kv_heads, head_dim, 0, write_kv=store)

        def project_encode_store(self, x, w_qkv, step, view, heads, kv_heads, head_dim):
            rt, (M, K) = self.rt, x.shape
            N = (heads + 2 * kv_heads) * head_dim
            plan = rt.qkv_plan(M, N, K)
            asked.append((M, plan))
            if x.dtype != torch.bfloat16 or plan is None:
                return super().project_encode_store(x, w_qkv, step, view, heads, kv_heads, head_dim)
            qkv = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
            common = (step.positions, step.token_seq, view.block_table(step), self.table, view.k, view.v, view.page_size,
                      heads, kv_heads, head_dim)
            if plan.kernel == "rows":
                return rt.ops.gemm_rows_qkv_rope(x, w_qkv.w, qkv, *common, write_kv=view.store, columns=plan.columns, rows=plan.rows)
            return rt.ops.gemv_qkv_rope(x, w_qkv.packed, qkv, *common, 0, write_kv=view.store)

    cfg = dict(architectures=["ToyStillLM"], width=256, inner=512, heads=4, kv_heads=2, head_dim=64, vocab=97, eps=1e-5)

    def plan(c, names=None):
        D = c["width"]
        norm = lambda n: PartSpec("rmsnorm", dict(width=D, eps=c["eps"]), dict(weight=n))
        layer = LayerPlan("pre_norm", position="still", mixer_norm=norm("n1"), ffn_norm=norm("n2"),
                          mixer=PartSpec("attention", dict(width=D, heads=c["heads"], kv_heads=c["kv_heads"], head_dim=c["head_dim"],
                                                           scale=c["head_dim"] ** -0.5), dict(q="q", k="k", v="v", o="o")),
                          feed_forward=PartSpec("swiglu", dict(width=D, inner=c["inner"]), dict(gate="gate", up="up", down="down")))
        return ModelPlan(vocab_size=c["vocab"], width=D, max_positions=1024, layers=[layer], order=[Place(0)],
                         embedding=PartSpec("table", dict(vocab=c["vocab"], width=D), dict(weight="emb")),
                         final_norm=norm("norm"), head=PartSpec("linear", dict(vocab=c["vocab"], width=D), dict(weight="emb")),
                         positions={"still": PartSpec("toy_still", dict(head_dim=c["head_dim"]))})

    registry.register_part("position", "toy_still", Still)
    registry.register_architecture(registry.Architecture("ToyStillLM", read_config=lambda d: d, plan=plan))
    g = torch.Generator().manual_seed(9)
    D, hd = cfg["width"], cfg["head_dim"]
    m = lambda *s: (torch.randn(*s, generator=g) * 0.06).bfloat16()
    t = {"emb": m(cfg["vocab"], D), "norm": torch.ones(D).bfloat16(), "n1": torch.ones(D).bfloat16(), "n2": torch.ones(D).bfloat16(),
         "q": m(cfg["heads"] * hd, D), "k": m(cfg["kv_heads"] * hd, D), "v": m(cfg["kv_heads"] * hd, D), "o": m(D, cfg["heads"] * hd),
         "gate": m(cfg["inner"], D), "up": m(cfg["inner"], D), "down": m(D, cfg["inner"])}
    json.dump(cfg, open(tmp_path / "config.json", "w"))
    st.write_file(str(tmp_path / "model.safetensors"), t.items())
    w = {k: v.double().numpy() for k, v in t.items()}

    def plain(tokens):
        h = w["emb"][np.asarray(tokens)][None]
        still = np.zeros(hd // 2)       # no turning at any position
        h = h + P.attention_layer(P.rms_norm(h, w["n1"], cfg["eps"]), w["q"], w["k"], w["v"], w["o"], cfg["heads"], cfg["kv_heads"], hd, still)
        h = h + P.swiglu_feed_forward(P.rms_norm(h, w["n2"], cfg["eps"]), w["gate"], w["up"], w["down"])
        return (P.rms_norm(h, w["norm"], cfg["eps"]) @ w["emb"].T)[0]

    eng = load_engine(str(tmp_path), dtype="bfloat16", max_tokens=300 * 64, max_seqs=300, graphs=False)
    rng = np.random.default_rng(4)
    for rows in (1, 9, 40, 100, 300):
        del asked[:]
        reqs = [[int(x) for x in rng.integers(0, cfg["vocab"], 3 + (5 * i) % 7)] for i in range(rows)]
        slots = [eng.open() for _ in reqs]
        eng.step([(s, r[:-1], []) for s, r in zip(slots, reqs)])
        got = eng.step([(s, [r[-1]], [0]) for s, r in zip(slots, reqs)]).double().cpu().numpy()    # one row per sequence
        assert asked[-1][0] == rows and asked[-1][1] == eng.rt.qkv_plan(rows, (cfg["heads"] + 2 * cfg["kv_heads"]) * hd, D)
        kind = asked[-1][1].kernel if asked[-1][1] is not None else None
        assert kind == {1: "packed", 9: "packed", 40: "rows", 100: "rows", 300: None}[rows], (rows, asked[-1])
        for i in range(0, rows, max(1, rows // 12)):
            want = plain(reqs[i])[-1]
            assert float(np.abs(got[i] - want).max() / np.abs(want).max()) <= 3e-2, (rows, i)
        for s in slots:
            eng.close(s)
