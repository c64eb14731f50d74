"""Other arrangements of a layer, defined here in the test and registered without a change to the
framework's files: a block with four norms around its two parts (a norm before and one after each),
a block that has a mixer and no feed-forward at all, and a block whose mixer and feed-forward read
the same normalised rows side by side.  The feed-forward of the first is a toy that
needs an integer table, which the random-weights mode makes from the toy architecture's own list of
checkpoint tensors.  The toy is no model of anyone's."""
import json

import numpy as np
import pytest
import torch

import plain_llama as P

TOY = dict(architectures=["ToyBlocksLM"], width=96, inner=136, heads=6, kv_heads=3, head_dim=16, vocab=203, eps=1e-5,
           theta=10000.0, max_positions=256)


def register_toy():
    import math
    from burn_lm_amd import registry
    from burn_lm_amd.models.plan import LayerPlan, ModelPlan, Place
    from burn_lm_amd.parts.base import Block, FeedForward, PartSpec, TensorSpec
    from burn_lm_amd.weights.random_init import IntegerTable, Normal

    class GatherFeedForward(FeedForward):
        """params: width.  names: table (integers), scale.  delta[:, j] = x[:, table[j]] * scale[j]."""

        def tensor_specs(self):
            D = self.params["width"]
            return {self.names["table"]: TensorSpec((D,), kind="int"), self.names["scale"]: TensorSpec((D,))}

        def bind(self, tensors, rt):
            self.rt = rt
            self.table = tensors[self.names["table"]].long()
            self.scale = tensors[self.names["scale"]].float()

        def forward(self, x, step):
            return (x.float()[:, self.table] * self.scale).to(self.rt.dtype)

    class SandwichBlock(Block):
        """h = x + post1(mixer(pre1(x))); y = h + post2(ffn(pre2(h)))."""
        roles = {"pre_mixer_norm": "norm", "mixer": "mixer", "post_mixer_norm": "norm",
                 "pre_ffn_norm": "norm", "feed_forward": "feed_forward", "post_ffn_norm": "norm"}

        def forward(self, h, delta, step, view):
            x = self.pre_mixer_norm.add_norm(h, delta)
            a = self.mixer.forward(x, step, view)
            if a.dim() == 3:
                a = a.sum(0)
            a = self.post_mixer_norm.add_norm(a.float().contiguous(), None, write_h=False)   # a norm of the delta alone
            x = self.pre_ffn_norm.add_norm(h, a)
            f = self.feed_forward.forward(x, step)
            return self.post_ffn_norm.add_norm(f.float().contiguous(), None, write_h=False)

    class ParallelBlock(Block):
        """y = x + mixer(norm(x)) + ffn(norm(x)): both parts read the same normalised rows; what they
        give is handed on as two float32 planes, which the next norm's add sums."""
        roles = {"norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}

        def forward(self, h, delta, step, view):
            x = self.norm.add_norm(h, delta)
            planes = []
            for d in (self.mixer.forward(x, step, view), self.feed_forward.forward(x, step)):
                planes += list(d.float()) if d.dim() == 3 else [d.float()]
            return torch.stack(planes).contiguous()

    class MixerOnlyBlock(Block):
        """y = x + mixer(norm(x)): a layer without a feed-forward."""
        roles = {"mixer_norm": "norm", "mixer": "mixer"}

        def forward(self, h, delta, step, view):
            return self.mixer.forward(self.mixer_norm.add_norm(h, delta), step, view)

    def plan(cfg, names=None):
        D = cfg["width"]
        norm = lambda n: PartSpec("rmsnorm", dict(width=D, eps=cfg["eps"]), dict(weight=n))
        attn = lambda i: PartSpec("attention", dict(width=D, heads=cfg["heads"], kv_heads=cfg["kv_heads"],
                                                    head_dim=cfg["head_dim"], scale=1 / math.sqrt(cfg["head_dim"])),
                                  dict(q=f"l{i}.q", k=f"l{i}.k", v=f"l{i}.v", o=f"l{i}.o"))
        layers = [LayerPlan("toy_sandwich", position="rope", pre_mixer_norm=norm("l0.n1"), mixer=attn(0),
                            post_mixer_norm=norm("l0.n2"), pre_ffn_norm=norm("l0.n3"),
                            feed_forward=PartSpec("toy_gather", dict(width=D), dict(table="l0.table", scale="l0.scale")),
                            post_ffn_norm=norm("l0.n4")),
                  LayerPlan("toy_mixer_only", {"mixer_norm": norm("l1.n1"), "mixer": attn(1)}, position="rope"),
                  LayerPlan("toy_parallel", position="rope", norm=norm("l2.n1"), mixer=attn(2),
                            feed_forward=PartSpec("swiglu", dict(width=D, inner=cfg["inner"]),
                                                  dict(gate="l2.gate", up="l2.up", down="l2.down")))]
        return ModelPlan(vocab_size=cfg["vocab"], width=D, max_positions=cfg["max_positions"],
                         embedding=PartSpec("table", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")),
                         layers=layers, order=[Place(0), Place(1), Place(2)], final_norm=norm("norm"),
                         head=PartSpec("linear", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")),
                         positions={"rope": PartSpec("rope", dict(head_dim=cfg["head_dim"], theta=cfg["theta"],
                                                                  pairing="interleaved", scaling=None))})

    def checkpoint_tensors(cfg):
        D, hd = cfg["width"], cfg["head_dim"]
        t = {"emb": ((cfg["vocab"], D), "table"), "norm": ((D,), "norm"), "l0.table": ((D,), IntegerTable(D)),
             "l0.scale": ((D,), Normal(std=0.5)), "l1.n1": ((D,), "norm"), "l2.n1": ((D,), "norm"),
             "l2.gate": ((cfg["inner"], D), "matrix"), "l2.up": ((cfg["inner"], D), "matrix"),
             "l2.down": ((D, cfg["inner"]), "matrix")}
        for n in ("n1", "n2", "n3", "n4"):
            t[f"l0.{n}"] = ((D,), "norm")
        for i in (0, 1, 2):
            t.update({f"l{i}.q": ((cfg["heads"] * hd, D), "matrix"), f"l{i}.k": ((cfg["kv_heads"] * hd, D), "matrix"),
                      f"l{i}.v": ((cfg["kv_heads"] * hd, D), "matrix"), f"l{i}.o": ((D, cfg["heads"] * hd), "matrix")})
        return t

    registry.register_part("feed_forward", "toy_gather", GatherFeedForward)
    registry.register_part("block", "toy_sandwich", SandwichBlock)
    registry.register_part("block", "toy_mixer_only", MixerOnlyBlock)
    registry.register_part("block", "toy_parallel", ParallelBlock)
    registry.register_architecture(registry.Architecture("ToyBlocksLM", read_config=lambda d: d, plan=plan,
                                                         checkpoint_tensors=checkpoint_tensors))


def toy_plain(tokens, w):
    c = TOY
    hd = c["head_dim"]
    freqs = P.rope_base_frequencies(hd, c["theta"])
    attn = lambda x, i: P.attention_layer(x, w[f"l{i}.q"], w[f"l{i}.k"], w[f"l{i}.v"], w[f"l{i}.o"],
                                          c["heads"], c["kv_heads"], hd, freqs)
    n = lambda x, name: P.rms_norm(x, w[name], c["eps"])
    h = w["emb"][np.asarray(tokens)][None]
    h = h + n(attn(n(h, "l0.n1"), 0), "l0.n2")
    x = n(h, "l0.n3")
    h = h + n(x[..., w["l0.table"].astype(np.int64)] * w["l0.scale"], "l0.n4")
    h = h + attn(n(h, "l1.n1"), 1)
    x = n(h, "l2.n1")
    h = h + attn(x, 2) + P.swiglu_feed_forward(x, w["l2.gate"], w["l2.up"], w["l2.down"])
    return (n(h, "norm") @ w["emb"].T)[0]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_a_block_with_four_norms_a_layer_without_a_feed_forward_and_a_parallel_block(tmp_path, dtype, tol):
    import burn_lm_amd
    from burn_lm_amd.engine.loading import load_engine
    from burn_lm_amd.weights import safetensors_io as st
    register_toy()
    folder = burn_lm_amd.write_random_model(str(tmp_path), TOY, seed=4, std=0.12, norm_jitter=0.1)
    f = st.open_folder(folder)
    stored = {n: f[n].tensor(n) for n in f}
    assert stored["l0.table"].dtype == torch.int32 and 0 <= int(stored["l0.table"].min()) and int(stored["l0.table"].max()) < TOY["width"]
    assert len(set(stored["l0.table"].tolist())) > TOY["width"] // 3      # a table of many different places
    w = {k: v.double().numpy() for k, v in stored.items()}
    eng = load_engine(folder, dtype=dtype, max_tokens=1024, max_seqs=4)
    kinds = [type(b).__name__ for b in eng.model.blocks]
    assert kinds == ["SandwichBlock", "MixerOnlyBlock", "ParallelBlock"] and not hasattr(eng.model.blocks[1], "feed_forward")
    assert [len(b.parts()) for b in eng.model.blocks] == [6, 2, 3]
    rng = np.random.default_rng(3)
    reqs = [[int(x) for x in rng.integers(0, TOY["vocab"], L)] for L in (130, 11, 66)]
    want = [toy_plain(r, w) for r in reqs]
    slots = [eng.open() for _ in reqs]
    cut = [len(r) - 5 for r in reqs]
    got = eng.step([(s, r[:k], list(range(k))) for s, r, k in zip(slots, reqs, cut)]).double().cpu().numpy()
    o = 0
    for i, k in enumerate(cut):
        for p in range(k):
            assert np.abs(got[o + p] - want[i][p]).max() / np.abs(want[i]).max() <= tol, (dtype, i, p)
        o += k
    for j in range(5):
        got = eng.step([(s, [r[k + j]], [0]) for s, r, k in zip(slots, reqs, cut)]).double().cpu().numpy()
        for i in range(3):
            assert np.abs(got[i] - want[i][cut[i] + j]).max() / np.abs(want[i]).max() <= tol, (dtype, i, cut[i] + j)
    for s in slots:
        eng.close(s)
    assert eng.cache.pages_in_use() == 0


def test_a_plan_that_names_a_role_its_block_does_not_have_is_refused(tmp_path):
    from burn_lm_amd import registry
    from burn_lm_amd.engine.model import Model
    from burn_lm_amd.parts.base import PartSpec
    register_toy()
    plan = registry.architecture("ToyBlocksLM").plan(TOY)
    plan.layers[1].parts["feed_forward"] = PartSpec("toy_gather", dict(width=TOY["width"]), dict(table="t", scale="s"))
    with pytest.raises(ValueError, match="no role 'feed_forward'"):
        Model(plan)
    plan = registry.architecture("ToyBlocksLM").plan(TOY)
    del plan.layers[0].parts["post_ffn_norm"]
    with pytest.raises(ValueError, match="lacks"):
        Model(plan)


# ---- a block whose two mixers each keep something: keys and values beside a fixed-size state ----------------------

HYBRID = dict(architectures=["ToyHybridLM"], width=80, inner=112, heads=5, kv_heads=5, head_dim=16, vocab=131, eps=1e-6,
              theta=5000.0, decay=0.7, max_positions=256)


def register_hybrid():
    import math
    from burn_lm_amd import registry
    from burn_lm_amd.models.plan import LayerPlan, ModelPlan, Place
    from burn_lm_amd.parts.base import Block, Mixer, PartSpec, StateNeed, TensorSpec

    class RunningSumMixer(Mixer):
        """params: width, decay.  names: w.  s_t = decay * s_{t-1} + x_t W, one float32 vector per sequence."""

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
            for slot, n in zip(step.host_slots, step.host_new):
                s = view.tensor[slot]
                for t in range(row, row + n):
                    s = self.a * s + u[t]
                    out[t] = s
                view.tensor[slot] = s
                row += n
            return out

    class HybridBlock(Block):
        """h = x + attention(norm(x)) + memory(norm(x)); y = h + ffn(ffn_norm(h)).  Both mixers keep
        something for every sequence, so the block asks the cache for two things."""
        roles = {"norm": "norm", "attention": "mixer", "memory": "mixer", "ffn_norm": "norm", "feed_forward": "feed_forward"}

        def cache_need(self):
            return (self.attention.cache_need(), self.memory.cache_need())

        def forward(self, h, delta, step, view):
            keys_and_values, state = view
            x = self.norm.add_norm(h, delta)
            planes = []
            for d in (self.attention.forward(x, step, keys_and_values), self.memory.forward(x, step, state)):
                planes += list(d.float()) if d.dim() == 3 else [d.float()]
            x = self.ffn_norm.add_norm(h, torch.stack(planes).contiguous())
            return self.feed_forward.forward(x, step)

    def plan(cfg, names=None):
        D = cfg["width"]
        norm = lambda n: PartSpec("rmsnorm", dict(width=D, eps=cfg["eps"]), dict(weight=n))
        attn = lambda i: PartSpec("attention", dict(width=D, heads=cfg["heads"], kv_heads=cfg["kv_heads"],
                                                    head_dim=cfg["head_dim"], scale=1 / math.sqrt(cfg["head_dim"])),
                                  dict(q=f"l{i}.q", k=f"l{i}.k", v=f"l{i}.v", o=f"l{i}.o"))
        ffn = lambda i: PartSpec("swiglu", dict(width=D, inner=cfg["inner"]),
                                 dict(gate=f"l{i}.gate", up=f"l{i}.up", down=f"l{i}.down"))
        layers = [LayerPlan("toy_hybrid", position="rope", norm=norm("l0.n1"), attention=attn(0),
                            memory=PartSpec("toy_running_sum", dict(width=D, decay=cfg["decay"]), dict(w="l0.w")),
                            ffn_norm=norm("l0.n2"), feed_forward=ffn(0)),
                  LayerPlan("pre_norm", position="rope", mixer_norm=norm("l1.n1"), mixer=attn(1), ffn_norm=norm("l1.n2"),
                            feed_forward=ffn(1))]
        # the hybrid layer runs twice; each run keeps keys, values and a state of its own
        return ModelPlan(vocab_size=cfg["vocab"], width=D, max_positions=cfg["max_positions"],
                         embedding=PartSpec("table", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")),
                         layers=layers, order=[Place(0), Place(1), Place(0)], final_norm=norm("norm"),
                         head=PartSpec("linear", dict(vocab=cfg["vocab"], width=D), dict(weight="emb")),
                         positions={"rope": PartSpec("rope", dict(head_dim=cfg["head_dim"], theta=cfg["theta"],
                                                                  pairing="interleaved", scaling=None))})

    def checkpoint_tensors(cfg):
        D, hd, I = cfg["width"], cfg["head_dim"], cfg["inner"]
        t = {"emb": ((cfg["vocab"], D), "table"), "norm": ((D,), "norm"), "l0.w": ((D, D), "matrix")}
        for i in (0, 1):
            t.update({f"l{i}.n1": ((D,), "norm"), f"l{i}.n2": ((D,), "norm"),
                      f"l{i}.q": ((cfg["heads"] * hd, D), "matrix"), f"l{i}.k": ((cfg["kv_heads"] * hd, D), "matrix"),
                      f"l{i}.v": ((cfg["kv_heads"] * hd, D), "matrix"), f"l{i}.o": ((D, cfg["heads"] * hd), "matrix"),
                      f"l{i}.gate": ((I, D), "matrix"), f"l{i}.up": ((I, D), "matrix"), f"l{i}.down": ((D, I), "matrix")})
        return t

    registry.register_part("mixer", "toy_running_sum", RunningSumMixer)
    registry.register_part("block", "toy_hybrid", HybridBlock)
    registry.register_architecture(registry.Architecture("ToyHybridLM", read_config=lambda d: d, plan=plan,
                                                         checkpoint_tensors=checkpoint_tensors))


def hybrid_plain(tokens, w):
    c = HYBRID
    freqs = P.rope_base_frequencies(c["head_dim"], c["theta"])
    attn = lambda x, i: P.attention_layer(x, w[f"l{i}.q"], w[f"l{i}.k"], w[f"l{i}.v"], w[f"l{i}.o"],
                                          c["heads"], c["kv_heads"], c["head_dim"], freqs)
    n = lambda x, name: P.rms_norm(x, w[name], c["eps"])
    ffn = lambda x, i: P.swiglu_feed_forward(x, w[f"l{i}.gate"], w[f"l{i}.up"], w[f"l{i}.down"])

    def running_sum(x):
        u = x @ w["l0.w"].T
        s, outs = np.zeros(c["width"]), []
        for t in range(u.shape[1]):
            s = c["decay"] * s + u[0, t]
            outs.append(s)
        return np.stack(outs)[None]

    def hybrid(h):
        x = n(h, "l0.n1")
        h = h + attn(x, 0) + running_sum(x)
        return h + ffn(n(h, "l0.n2"), 0)

    h = hybrid(w["emb"][np.asarray(tokens)][None])
    h = h + attn(n(h, "l1.n1"), 1)
    h = h + ffn(n(h, "l1.n2"), 1)
    h = hybrid(h)
    return (n(h, "norm") @ w["emb"].T)[0]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_a_block_whose_two_mixers_keep_keys_and_values_and_a_state(tmp_path, dtype, tol):
    import burn_lm_amd
    from burn_lm_amd.cache.cache import KVView, StateView
    from burn_lm_amd.engine.loading import load_engine
    from burn_lm_amd.weights import safetensors_io as st
    register_hybrid()
    folder = burn_lm_amd.write_random_model(str(tmp_path), HYBRID, seed=9, std=0.1, norm_jitter=0.1)
    f = st.open_folder(folder)
    w = {n: f[n].tensor(n).double().numpy() for n in f}
    eng = load_engine(folder, dtype=dtype, max_tokens=768, max_seqs=3)
    views = eng.cache.views
    assert [type(v) for v in views] == [tuple, KVView, tuple]
    for v in (views[0], views[2]):
        assert isinstance(v[0], KVView) and isinstance(v[1], StateView)
    # three places keep keys and values of one shape: one group, three planes; two states of their own
    assert len(eng.cache.groups) == 1 and eng.cache.groups[0].k_storage.shape[0] == 3
    assert views[0][1].tensor.data_ptr() != views[2][1].tensor.data_ptr()
    rng = np.random.default_rng(12)
    for batch in ([70, 9, 33], [41, 100]):            # the second batch takes the slots and pages of the first
        reqs = [[int(x) for x in rng.integers(0, HYBRID["vocab"], L)] for L in batch]
        want = [hybrid_plain(r, w) for r in reqs]
        slots = [eng.open() for _ in reqs]
        cut = [len(r) - 4 for r in reqs]
        got = eng.step([(s, r[:k], [0, k - 1]) for s, r, k in zip(slots, reqs, cut)]).double().cpu().numpy()
        for i, k in enumerate(cut):
            for j, p in enumerate((0, k - 1)):
                assert np.abs(got[2 * i + j] - want[i][p]).max() / np.abs(want[i]).max() <= tol, (dtype, batch, i, p)
        for j in range(4):
            got = eng.step([(s, [r[k + j]], [0]) for s, r, k in zip(slots, reqs, cut)]).double().cpu().numpy()
            for i in range(len(reqs)):
                assert np.abs(got[i] - want[i][cut[i] + j]).max() / np.abs(want[i]).max() <= tol, (dtype, batch, i, cut[i] + j)
        for s in slots:
            eng.close(s)
        assert eng.cache.pages_in_use() == 0
