"""Each part alone against the plain implementation, and the generality of the assembly: a toy architecture
defined here (a mixer with state of its own, a routed feed-forward, another position encoding, a windowed
layer, a layer that runs twice, a run that reads another run's cache) is registered, written to a model
folder, loaded by name and stepped in portions, without touching the framework's files."""
import math

import numpy as np
import pytest
import torch

from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def fw():
    import llm_infrence_engine_amd as root
    from llm_infrence_engine_amd import cache, config, engine, parts, weights
    from llm_infrence_engine_amd.kernels import ops

    class NS:
        pass
    ns = NS()
    ns.root, ns.cache, ns.config, ns.engine, ns.parts, ns.weights, ns.ops = root, cache, config, engine, parts, weights, ops
    return ns


def rt_for(fw, dtype):
    return fw.parts.Runtime(torch.device(DEV), dtype)


def getter(tensors, fw, rt):
    return lambda spec: fw.weights.place(tensors[spec.name], spec, rt.dtype, rt.device)


def random_for(part, seed, fw, std=0.3):
    return fw.weights.random_tensors(part.tensor_specs(), seed, std=std, dtype="float32")


# ------------------------------------------------------------------------------------------------ parts alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(fw, dtype):
    part = fw.parts.build_part("norm", fw.config.PartSpec("rms_norm", "n.", {"size": 200, "eps": 3e-4}))
    t = random_for(part, 0, fw)
    rt = rt_for(fw, dtype)
    part.load(getter(t, fw, rt), rt)
    x = torch.randn(6, 200, device=DEV) * 2
    want = P.rms_norm(x.double().cpu(), t["n.weight"].double(), 3e-4)
    got = part.forward(x)
    assert got.dtype == dtype
    torch.testing.assert_close(got.double().cpu(), want, atol=2e-5 if dtype == torch.float32 else 3e-2, rtol=1e-2)


def test_feed_forward_part(fw):
    part = fw.parts.build_part("feed_forward", fw.config.PartSpec("swiglu", "m.", {"hidden_size": 72, "intermediate_size": 200}))
    t = random_for(part, 1, fw, std=0.2)
    rt = rt_for(fw, torch.float32)
    part.load(getter(t, fw, rt), rt)
    h = torch.randn(5, 72, device=DEV)
    want = P.swiglu_mlp(h.double().cpu(), {k: v.double() for k, v in t.items()}, "m.")
    torch.testing.assert_close(part.forward(h, None).double().cpu(), want, atol=1e-4, rtol=1e-4)


def test_embedding_and_head_parts(fw):
    emb = fw.parts.build_part("embedding", fw.config.PartSpec("token_embedding", "e.", {"vocab_size": 331, "hidden_size": 72}))
    head = fw.parts.build_part("head", fw.config.PartSpec("lm_head", "h.", {"hidden_size": 72, "vocab_size": 331, "tied_to": "e.weight"}))
    t = random_for(emb, 2, fw)
    rt = rt_for(fw, torch.bfloat16)
    placed = {}

    def get(spec):
        if spec.name not in placed:
            placed[spec.name] = fw.weights.place(t[spec.name], spec, rt.dtype, rt.device)
        return placed[spec.name]
    emb.load(get, rt); head.load(get, rt)
    assert head.weight.data_ptr() == emb.weight.data_ptr()     # tied: one matrix (the reference's tests/test_model_parity.py:29-31)
    assert head.ignorable() == ["h.weight"]

    class Ctx:
        num_tokens = 4
        token_ids = torch.tensor([0, 330, 7, 7], dtype=torch.int32, device=DEV)
    x = emb.forward(Ctx)
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), t["e.weight"].bfloat16().float()[[0, 330, 7, 7]])
    h = torch.randn(3, 72, device=DEV).bfloat16()
    logits = head.forward(h)
    assert logits.dtype == torch.float32 and logits.shape == (3, 331)
    torch.testing.assert_close(logits.cpu().double(), h.double().cpu() @ t["e.weight"].bfloat16().double().T, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("nh,nkv,d,window,page_size", [(6, 2, 32, None, 8), (5, 5, 48, 9, 4), (4, 1, 16, None, 16)])
def test_attention_part_in_portions(fw, nh, nkv, d, window, page_size):
    """The mixer alone, fed 50 tokens as 23 + 2 + 24 + 1, against the plain attention block."""
    H, T = 40, 50
    pos = fw.parts.build_part("position", fw.config.PartSpec("rotary_half", "", {"head_dim": d, "rotary_dim": d, "theta": 500.0}))
    spec = fw.config.PartSpec("gqa_attention", "a.", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                                      "scale": 1 / math.sqrt(d), "qkv_bias": True, "out_bias": False, "window": window})
    part = fw.parts.build_part("mixer", spec, position=pos)
    t = random_for(part, 3, fw, std=0.4)
    rt = rt_for(fw, torch.float32)
    part.load(getter(t, fw, rt), rt)
    assert part.cache_need() == fw.parts.KVNeed(nkv, d, window, 16, torch.bfloat16)    # loaded or not, whatever the type
    h = torch.randn(T, H)
    w = {k: v.double() for k, v in t.items()}
    cfg = {"num_heads": nh, "num_kv_heads": nkv, "head_dim": d}
    cos, sin = P.rope_cos_sin(torch.arange(T), d, 500.0)
    if window is None:
        want = P.attention_block(h.double(), w, "a.", cfg, cos, sin)
    else:  # the plain block has no window: assemble it from the plain pieces
        q = (h.double() @ w["a.q_proj.weight"].T + w["a.q_proj.bias"]).view(T, nh, d).transpose(0, 1)
        k = (h.double() @ w["a.k_proj.weight"].T + w["a.k_proj.bias"]).view(T, nkv, d).transpose(0, 1)
        v = (h.double() @ w["a.v_proj.weight"].T + w["a.v_proj.bias"]).view(T, nkv, d).transpose(0, 1)
        o = P.causal_attention(P.apply_rope(q, cos, sin), P.apply_rope(k, cos, sin), v, window=window)
        want = o.transpose(0, 1).reshape(T, nh * d) @ w["a.o_proj.weight"].T
    layout = fw.cache.CacheLayout([(part.cache_need(), None, None)])
    m = fw.cache.CacheManager(layout, page_size, 20, 2, 64)
    pools = fw.cache.CachePools(layout, page_size, 20, 2, rt, m.max_pages_per_request)
    for t in pools.pages[0].values():
        t.fill_(1e4)                                         # what a reused page may hold must not matter
    builder = fw.engine.BatchBuilder(m, pools, 1000, rt.device)
    m.add("other")                                           # so that the request's table row is not row 0
    m.add("x")
    got, p = [], 0
    for n in (23, 2, 24, 1):
        m.grow("x", p + n)
        b = builder.build([fw.engine.StepEntry("x", [1] * n, [])])
        ctx = b.ctx
        got.append(part.forward(h[p:p + n].to(DEV), ctx, pools.kv_view(0, ctx.state_slots, b.slots[0]), None).cpu())
        p += n
        m.advance("x", p)
    torch.testing.assert_close(torch.cat(got).double(), want, atol=2e-4, rtol=2e-4)


# ------------------------------------------------------------------------------------------------ a toy architecture
def register_toys(fw):
    from dataclasses import dataclass

    parts, cfgm, ops = fw.parts, fw.config, fw.ops
    TensorSpec = fw.weights.TensorSpec

    class ToyDecay(parts.Mixer):
        """state <- decay * state + W_in h_t ; seen <- seen + 1 ; out_t = W_out state / (1 + seen / 100)
        Two states of fixed size per request, of different types.  Single tokens are handled with device tensors
        only, so a decode step of this mixer can be captured into a graph; portions walk the requests on the host."""

        graph_safe = "decode"

        def __init__(self, prefix, position, hidden_size, state_size, decay):
            self.prefix, self.H, self.S, self.decay = prefix, hidden_size, state_size, decay

        def tensor_specs(self):
            return [TensorSpec(self.prefix + "in.weight", (self.S, self.H)), TensorSpec(self.prefix + "out.weight", (self.H, self.S))]

        def load(self, get, rt):
            self.rt = rt
            self.w_in, self.w_out = (get(s).float().contiguous() for s in self.tensor_specs())

        def state_need(self):
            return (parts.StateNeed((self.S,), torch.float32), parts.StateNeed((), torch.int32))

        def forward(self, h, ctx, kv, state):
            assert kv is None
            s_all, seen_all = state.slots
            hin = ops.gemm_generic(h.float().contiguous(), self.w_in, torch.empty(h.shape[0], self.S, device=h.device))
            if ctx.decode_only:                       # one token per request: no look at the host copies
                idx = ctx.state_slots.long()
                s = self.decay * s_all.index_select(0, idx) + hin
                seen = seen_all.index_select(0, idx) + 1
                s_all.index_copy_(0, idx, s)
                seen_all.index_copy_(0, idx, seen)
                out = ops.gemm_generic(s, self.w_out, torch.empty(h.shape[0], self.H, device=h.device))
                return (out / (1 + seen.float() / 100)[:, None]).to(h.dtype)
            out = torch.empty_like(h)
            o = 0
            for n, slot in zip(ctx.q_lens_host, ctx.state_slots_host):
                s, seen = s_all[slot].clone(), int(seen_all[slot])
                for t in range(n):
                    s = self.decay * s + hin[o + t]
                    seen += 1
                    out[o + t] = ((self.w_out @ s) / (1 + seen / 100)).to(h.dtype)
                s_all[slot] = s
                seen_all[slot] = seen
                o += n
            return out

    class ToyLatent(parts.Mixer):
        """One head of attention over a cache that holds one tensor per token: the latent c_t = W_c h_t, from which
        keys W_k c and values W_v c are made when they are read."""

        graph_safe = False      # walks the requests on the host

        def __init__(self, prefix, position, hidden_size, latent_size, key_size):
            self.prefix, self.H, self.r, self.dk = prefix, hidden_size, latent_size, key_size

        def tensor_specs(self):
            p = self.prefix
            return [TensorSpec(p + "c.weight", (self.r, self.H)), TensorSpec(p + "q.weight", (self.dk, self.H)),
                    TensorSpec(p + "k.weight", (self.dk, self.r)), TensorSpec(p + "v.weight", (self.H, self.r))]

        def load(self, get, rt):
            self.rt = rt
            self.wc, self.wq, self.wk, self.wv = (get(s).float() for s in self.tensor_specs())

        def cache_need(self):
            return parts.CacheNeed((parts.PageTensor("latent", 1, self.r),), None)

        def forward(self, h, ctx, kv, state):
            x = h.float()
            pages = kv.pages["latent"]                                # [pages, 1, page_size, r]
            flat = pages.view(-1, self.r)
            flat[kv.slot_mapping.long()] = (x @ self.wc.T).to(flat.dtype)
            q = x @ self.wq.T
            out = torch.empty_like(x)
            o = 0
            for r, (n, start) in enumerate(zip(ctx.q_lens_host, ctx.start_pos_host)):
                held = -(-(start + n) // pages.shape[2])
                c = pages[kv.pages_of(r)[:held].long()].reshape(-1, self.r)[:start + n].float()
                scores = (q[o:o + n] @ (c @ self.wk.T).T) / math.sqrt(self.dk)
                j = torch.arange(start + n, device=x.device)[None, :]
                i = torch.arange(start, start + n, device=x.device)[:, None]
                scores = scores.masked_fill(j > i, float("-inf"))
                out[o:o + n] = scores.softmax(-1) @ (c @ self.wv.T)
                o += n
            return out.to(h.dtype)

    class ToyRouted(parts.FeedForward):
        """router logits in float -> softmax -> the best expert alone, weighted by its probability"""

        graph_safe = False      # waits for the device to learn which experts have rows

        def __init__(self, prefix, hidden_size, intermediate_size, num_experts):
            self.prefix, self.H, self.I, self.E = prefix, hidden_size, intermediate_size, num_experts

        def tensor_specs(self):
            return [TensorSpec(self.prefix + "router.weight", (self.E, self.H), keep32=True),
                    TensorSpec(self.prefix + "up.weight", (self.E * self.I, self.H)),
                    TensorSpec(self.prefix + "down.weight", (self.E * self.H, self.I))]

        def load(self, get, rt):
            self.rt = rt
            self.router, self.up, self.down = (get(s).float() for s in self.tensor_specs())

        def forward(self, h, ctx):
            x = h.float()
            prob = (x @ self.router.T).softmax(-1)
            best = prob.argmax(-1)
            out = torch.zeros_like(x)
            for e in range(self.E):
                rows = (best == e).nonzero().flatten()
                if rows.numel():
                    a = torch.relu(x[rows] @ self.up[e * self.I:(e + 1) * self.I].T)
                    out[rows] = (a @ self.down[e * self.H:(e + 1) * self.H].T) * prob[rows, e:e + 1]
            return out.to(h.dtype)

    class ToyOffset(parts.PositionEncoding):
        """adds table[position % period] to every q and k head (absolute, not rotary)"""

        def __init__(self, prefix, head_dim, period):
            self.prefix, self.d, self.period = prefix, head_dim, period

        def tensor_specs(self):
            return [TensorSpec(self.prefix + "table", (self.period, self.d))]

        def load(self, get, rt):
            self.rt = rt
            self.table = get(self.tensor_specs()[0])

        def encode_and_store(self, qkv, nh, nkv, d, ctx, kv):
            v = qkv.view(qkv.shape[0], nh + 2 * nkv, d)
            v[:, :nh + nkv] += self.table[(ctx.positions.long() % self.period)][:, None, :]
            if kv is not None and kv.store:
                ops.rope_store(qkv, nh, nkv, d, 0, None, None, kv.slot_mapping, kv.k_pages, kv.v_pages, kv.v_transposed)

    class ToySandwich(parts.Block):
        """Four norms to a layer: x += post_a(mixer(pre_a(x))); x += post_f(feed_forward(pre_f(x)))."""

        takes = {"pre_mixer_norm": "norm", "mixer": "mixer", "post_mixer_norm": "norm", "pre_ff_norm": "norm",
                 "feed_forward": "feed_forward", "post_ff_norm": "norm"}

        def forward(self, x, pending, ctx, kv, state):
            if pending is not None:
                ops.residual_add(x, pending)
            a = self.mixer.forward(self.pre_mixer_norm.forward(x), ctx, kv, state)
            ops.residual_add(x, self.post_mixer_norm.forward(a.float().contiguous()))
            f = self.feed_forward.forward(self.pre_ff_norm.forward(x), ctx)
            return self.post_ff_norm.forward(f.float().contiguous())       # the next norm adds it

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        width: int
        heads: int
        kv_heads: int
        head_size: int
        inner: int
        experts: int
        state_size: int
        decay: float
        window: int
        eps: float
        latent: int = 12
        capturable: bool = False     # only parts that a graph can hold: attention, the decaying state, dense feed-forwards

        @classmethod
        def from_dict(cls, d):
            return cls(**{k: d[k] for k in cls.__dataclass_fields__})

        def to_dict(self):
            d = {k: getattr(self, k) for k in self.__dataclass_fields__}
            d["architectures"] = ["ToyForCausalLM"]
            return d

        def to_spec(self):
            H, d = self.width, self.head_size
            PartSpec, layer, Run = cfgm.PartSpec, cfgm.layer, cfgm.Run
            norm = lambda p: PartSpec("rms_norm", p, {"size": H, "eps": self.eps})

            def attn(p, window, position):
                return dict(mixer=PartSpec("gqa_attention", p + "attn.", {
                    "hidden_size": H, "num_heads": self.heads, "num_kv_heads": self.kv_heads, "head_dim": d,
                    "scale": 1 / math.sqrt(d), "qkv_bias": False, "out_bias": True, "window": window}), position=position)
            rotary = PartSpec("rotary_half", "", {"head_dim": d, "rotary_dim": d // 2, "theta": 100.0})
            dense = lambda p: PartSpec("swiglu", p + "ff.", {"hidden_size": H, "intermediate_size": self.inner})
            routed = lambda p: PartSpec("toy_routed", p + "ff.", {"hidden_size": H, "intermediate_size": self.inner, "num_experts": self.experts})
            decay = dict(mixer=PartSpec("toy_decay", "l1.mix.", {"hidden_size": H, "state_size": self.state_size, "decay": self.decay}))
            head = PartSpec("lm_head", "head.", {"hidden_size": H, "vocab_size": self.vocab_size, "tied_to": None})
            emb = PartSpec("token_embedding", "emb.", {"vocab_size": self.vocab_size, "hidden_size": H})
            if self.capturable:
                layers = [layer("pre_norm_residual", feed_forward=dense(f"l{i}."), mixer_norm=norm(f"l{i}.n1."),
                                feed_forward_norm=norm(f"l{i}.n2."), **mix)
                          for i, mix in enumerate([attn("l0.", None, rotary), decay])]
                return cfgm.ModelSpec("ToyForCausalLM", H, self.vocab_size, emb, tuple(layers), (Run(0), Run(1), Run(1)),
                                      norm("final."), head)
            layers = []
            for i, (mix, ff) in enumerate([
                    (attn("l0.", self.window, rotary), dense("l0.")),
                    (decay, routed("l1.")),
                    (attn("l2.", None, PartSpec("toy_offset", "l2.pos.", {"head_dim": d, "period": 7})), routed("l2.")),
                    (attn("l3.", self.window - 1, rotary), dense("l3."))]):
                p = f"l{i}."
                layers.append(layer("pre_norm_residual", feed_forward=ff, mixer_norm=norm(p + "n1."),
                                    feed_forward_norm=norm(p + "n2."), **mix))
            layers.append(layer("toy_sandwich", pre_mixer_norm=norm("l4.n1."), post_mixer_norm=norm("l4.n2."),
                                pre_ff_norm=norm("l4.n3."), post_ff_norm=norm("l4.n4."), feed_forward=dense("l4."),
                                mixer=PartSpec("toy_latent", "l4.mix.", {"hidden_size": H, "latent_size": self.latent, "key_size": 8})))
            # layer 1 runs twice (two states), run 4 reads the keys and values that run 0 stored, the last layer
            # has four norms and a cache of one tensor per token
            order = (Run(0), Run(1), Run(2), Run(1), Run(3, cache_of=0), Run(4))
            return cfgm.ModelSpec("ToyForCausalLM", H, self.vocab_size, emb, tuple(layers), order, norm("final."), head)

    parts.register_part("mixer", "toy_decay", ToyDecay)
    parts.register_part("mixer", "toy_latent", ToyLatent)
    parts.register_part("feed_forward", "toy_routed", ToyRouted)
    parts.register_part("position", "toy_offset", ToyOffset)
    parts.register_part("block", "toy_sandwich", ToySandwich)
    cfgm.register_architecture("ToyForCausalLM", ToyConfig)
    return ToyConfig


def toy_plain(w, c, ids):
    """The toy model whole, in double, written out here from the toy parts' one-line definitions."""
    T, H, d, nh, nkv = len(ids), c.width, c.head_size, c.heads, c.kv_heads
    x = w["emb.weight"][ids]
    pos = torch.arange(T)
    cos, sin = P.rope_cos_sin(pos, d // 2, 100.0)

    def rot(t):  # partial rotary: the first half of each head
        return torch.cat((P.apply_rope(t[..., :d // 2], cos, sin), t[..., d // 2:]), -1)

    def attn(h, p, window, position, kv=None):
        q = (h @ w[p + "attn.q_proj.weight"].T).view(T, nh, d).transpose(0, 1)
        k = (h @ w[p + "attn.k_proj.weight"].T).view(T, nkv, d).transpose(0, 1)
        v = (h @ w[p + "attn.v_proj.weight"].T).view(T, nkv, d).transpose(0, 1)
        if position == "rotary":
            q, k = rot(q), rot(k)
        else:
            off = w["l2.pos.table"][pos % 7]
            q, k = q + off, k + off
        if kv is not None:
            k, v = kv
        o = P.causal_attention(q, k, v, window=window).transpose(0, 1).reshape(T, nh * d)
        return o @ w[p + "attn.o_proj.weight"].T + w[p + "attn.o_proj.bias"], (k, v)

    def decay(h):
        s = torch.zeros(c.state_size, dtype=h.dtype)
        out = []
        for t in range(T):
            s = c.decay * s + w["l1.mix.in.weight"] @ h[t]
            out.append((w["l1.mix.out.weight"] @ s) / (1 + (t + 1) / 100))
        return torch.stack(out)

    def latent(h):
        cl = h @ w["l4.mix.c.weight"].T
        q, k, v = h @ w["l4.mix.q.weight"].T, cl @ w["l4.mix.k.weight"].T, cl @ w["l4.mix.v.weight"].T
        return P.causal_attention(q[None], k[None], v[None])[0]          # one head, scale 1 / sqrt(key size)

    def dense(h, p):
        return P.swiglu_mlp(h, {"gate_proj.weight": w[p + "ff.gate_proj.weight"], "up_proj.weight": w[p + "ff.up_proj.weight"],
                                "down_proj.weight": w[p + "ff.down_proj.weight"]}, "")

    def routed(h, p):
        prob = (h @ w[p + "ff.router.weight"].T).softmax(-1)
        best = prob.argmax(-1)
        out = torch.zeros_like(h)
        for t in range(T):
            e = int(best[t])
            a = torch.relu(w[p + "ff.up.weight"][e * c.inner:(e + 1) * c.inner] @ h[t])
            out[t] = (w[p + "ff.down.weight"][e * H:(e + 1) * H] @ a) * prob[t, e]
        return out

    n = lambda t, p: P.rms_norm(t, w[p + "weight"], c.eps)
    if c.capturable:
        a, _ = attn(n(x, "l0.n1."), "l0.", None, "rotary"); x = x + a
        x = x + dense(n(x, "l0.n2."), "l0.")
        for _ in range(2):
            x = x + decay(n(x, "l1.n1.")); x = x + dense(n(x, "l1.n2."), "l1.")
        return n(x, "final.") @ w["head.weight"].T
    a, kv0 = attn(n(x, "l0.n1."), "l0.", c.window, "rotary"); x = x + a
    x = x + dense(n(x, "l0.n2."), "l0.")
    x = x + decay(n(x, "l1.n1.")); x = x + routed(n(x, "l1.n2."), "l1.")
    a, _ = attn(n(x, "l2.n1."), "l2.", None, "offset"); x = x + a
    x = x + routed(n(x, "l2.n2."), "l2.")
    x = x + decay(n(x, "l1.n1.")); x = x + routed(n(x, "l1.n2."), "l1.")
    a, _ = attn(n(x, "l3.n1."), "l3.", c.window - 1, "rotary", kv=kv0); x = x + a
    x = x + dense(n(x, "l3.n2."), "l3.")
    x = x + n(latent(n(x, "l4.n1.")), "l4.n2.")
    x = x + n(dense(n(x, "l4.n3."), "l4."), "l4.n4.")
    return n(x, "final.") @ w["head.weight"].T


def test_toy_architecture_is_registered_built_and_stepped(fw, tmp_path):
    ToyConfig = register_toys(fw)
    cfg = ToyConfig(vocab_size=101, width=40, heads=4, kv_heads=2, head_size=16, inner=56, experts=3, state_size=24,
                    decay=0.8, window=6, eps=1e-5)
    d = fw.root.write_random_model(tmp_path / "toy", cfg, seed=4, dtype="float32", std=0.25)
    assert type(fw.root.load_config(d)).__name__ == "ToyConfig"
    runner = fw.engine.load_runner(d, dtype="float32", page_size=4, num_pages=40, max_requests=3, max_len=64, hip_graphs=True)
    assert runner.graphs is None            # the routed feed-forward and the latent mixer cannot be captured, and say so
    lay = runner.layout
    assert len(lay.group_keys) == 3 and lay.state_runs == [1, 3]
    assert lay.run_stores == [True, False, True, False, False, True]
    assert lay.run_group[4] == lay.run_group[0] and lay.run_entry[4] == lay.run_entry[0]
    assert [t.name for t in lay.group_keys[lay.run_group[5]].tensors] == ["latent"]
    assert sorted(runner.pools.pages[lay.run_group[5]]) == ["latent"] and len(runner.pools.state[1]) == 2
    assert runner.manager.bytes_per_token(4) == 4 * (2 * 2 * 2 * 16 + 12)     # two attention caches of k and v, one latent
    w = P.read_weights(d, torch.float64)
    rng = np.random.default_rng(0)
    seqs = {r: [int(t) for t in rng.integers(0, 101, n)] for r, n in (("a", 37), ("b", 22), ("c", 9))}
    want = {r: toy_plain(w, cfg, torch.tensor(t)).numpy() for r, t in seqs.items()}
    Entry = fw.engine.StepEntry
    # a whole; then b and c in portions beside each other, with a's slot and pages used again by c
    got = runner.step([Entry("a", seqs["a"], list(range(37)))]).cpu().numpy()
    assert np.abs(got - want["a"]).max() < 1e-3
    runner.free_request("a")
    out = {"b": [], "c": []}
    cuts = {"b": [5, 2, 14, 1], "c": [2, 6, 1]}
    pos = {"b": 0, "c": 0}
    for i in range(4):
        entries = []
        for r in ("b", "c"):
            if i < len(cuts[r]):
                n = cuts[r][i]
                entries.append(Entry(r, seqs[r][pos[r]:pos[r] + n], list(range(n))))
        logits = runner.step(entries).cpu().numpy()
        o = 0
        for e in entries:
            out[e.req_id].append(logits[o:o + len(e.tokens)])
            o += len(e.tokens)
            pos[e.req_id] += len(e.tokens)
        runner.manager.check_invariants()
    for r in ("b", "c"):
        assert np.abs(np.concatenate(out[r]) - want[r]).max() < 1e-3, r
    # the windowed group has given pages back along the way; the groups that keep everything have not
    held = runner.manager.pages_held("b")
    for g, key in enumerate(lay.group_keys):
        assert (len(held[g]) == 6) == (key.window is None)
    runner.free_request("b"); runner.free_request("c")
    assert all(g.allocator.num_in_use() == 0 for g in runner.manager.groups)


def test_a_layer_with_two_caching_mixers(fw, tmp_path):
    """An arrangement of its own with two attention mixers of different head counts and sizes side by side: the
    layer's cache need holds both their page tensors under the parts' names, each mixer is handed its own, the
    model decodes from graphs in bfloat16 and follows the plain computation in both types."""
    from dataclasses import dataclass

    parts, cfgm, ops = fw.parts, fw.config, fw.ops

    class Twin(parts.Block):
        """x += wide(norm(x)) + narrow(norm(x))"""

        takes = {"norm": "norm", "wide": "mixer", "narrow": "mixer"}

        def forward(self, x, pending, ctx, kv, state):
            if pending is not None:
                ops.residual_add(x, pending)
            h = self.norm.forward(x)
            a = self.wide.forward(h, ctx, self.kv_of("wide", kv), None)
            b = self.narrow.forward(h, ctx, self.kv_of("narrow", kv), None)
            ops.residual_add(x, a)
            return b                                   # the next norm (or the head's) adds it

    @dataclass(frozen=True)
    class TwinConfig:
        vocab_size: int = 90
        width: int = 64

        @classmethod
        def from_dict(cls, d):
            return cls(d["vocab_size"], d["width"])

        def to_dict(self):
            return {"vocab_size": self.vocab_size, "width": self.width, "architectures": ["TwinForCausalLM"]}

        def to_spec(self):
            H = self.width
            PartSpec = cfgm.PartSpec

            def attn(p, nh, nkv, d):
                return PartSpec("gqa_attention", p, {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                                      "scale": d ** -0.5, "qkv_bias": True, "out_bias": False, "window": None})
            layers = tuple(cfgm.layer("twin", norm=PartSpec("rms_norm", f"l{i}.n.", {"size": H, "eps": 1e-6}),
                                      wide=attn(f"l{i}.wide.", 4, 2, 32), narrow=attn(f"l{i}.narrow.", 2, 1, 64))
                           for i in range(2))
            return cfgm.ModelSpec("TwinForCausalLM", H, self.vocab_size,
                                  PartSpec("token_embedding", "emb.", {"vocab_size": self.vocab_size, "hidden_size": H}),
                                  layers, (cfgm.Run(0), cfgm.Run(1)), PartSpec("rms_norm", "final.", {"size": H, "eps": 1e-6}),
                                  PartSpec("lm_head", "head.", {"hidden_size": H, "vocab_size": self.vocab_size, "tied_to": None}))

    parts.register_part("block", "twin", Twin)
    cfgm.register_architecture("TwinForCausalLM", TwinConfig)
    cfg = TwinConfig()
    d = fw.root.write_random_model(tmp_path / "twin", cfg, seed=8, dtype="float32", std=0.2)
    w = P.read_weights(d, torch.float64)

    def plain(ids):
        T = len(ids)
        x = w["emb.weight"][ids]
        for i in range(2):
            h = P.rms_norm(x, w[f"l{i}.n.weight"], 1e-6)
            for name, nh, nkv, hd in (("wide", 4, 2, 32), ("narrow", 2, 1, 64)):
                p = f"l{i}.{name}."
                q = (h @ w[p + "q_proj.weight"].T + w[p + "q_proj.bias"]).view(T, nh, hd).transpose(0, 1)
                k = (h @ w[p + "k_proj.weight"].T + w[p + "k_proj.bias"]).view(T, nkv, hd).transpose(0, 1)
                v = (h @ w[p + "v_proj.weight"].T + w[p + "v_proj.bias"]).view(T, nkv, hd).transpose(0, 1)
                o = P.causal_attention(q, k, v).transpose(0, 1).reshape(T, nh * hd)     # no position encoding
                x = x + o @ w[p + "o_proj.weight"].T
        return P.rms_norm(x, w["final.weight"], 1e-6) @ w["head.weight"].T

    rng = np.random.default_rng(2)
    seq = [int(t) for t in rng.integers(0, 90, 45)]
    want = plain(torch.tensor(seq)).numpy()
    Entry = fw.engine.StepEntry
    for dtype, bound in (("float32", 1e-3), ("bfloat16", 0.15)):
        runner = fw.engine.load_runner(d, dtype=dtype, page_size=16, num_pages=8, max_requests=2, max_len=64,
                                       hip_graphs=dtype == "bfloat16")
        need = runner.model.layers[0].cache_need()
        assert [t.name for t in need.tensors] == ["wide.k", "wide.v", "narrow.k", "narrow.v"]
        assert [(t.heads, t.width) for t in need.tensors] == [(2, 32), (2, 32), (1, 64), (1, 64)]
        assert len(runner.layout.group_keys) == 1 and runner.manager.bytes_per_token(1) == 2 * (2 * 2 * 32 + 2 * 64)
        got = [runner.step([Entry("x", seq[:30], list(range(30)))]).float().cpu().numpy()]
        for t in range(30, 45):
            got.append(runner.step([Entry("x", [seq[t]], [0])]).float().cpu().numpy())
        assert np.abs(np.concatenate(got) - want).max() < bound, dtype
        if dtype == "bfloat16":
            assert runner.graphs is not None and runner.graphs.launches == 16
    # mixers that keep their tokens for different spans cannot share a layer
    bad = Twin.build({"norm": cfg.to_spec().layers[0].parts["norm"], "wide": cfg.to_spec().layers[0].parts["wide"],
                      "narrow": cfgm.PartSpec("gqa_attention", "n.", {"hidden_size": 64, "num_heads": 2, "num_kv_heads": 1,
                                                                    "head_dim": 64, "scale": 0.125, "window": 7})})
    with pytest.raises(ValueError, match="different spans"):
        bad.cache_need()


def test_a_mixer_with_state_that_says_so_decodes_from_graphs(fw, tmp_path):
    """The decaying-state mixer handles single tokens with device tensors only and declares ``graph_safe``: a model of
    it, attention and dense feed-forwards decodes from captured graphs, several steps to a launch too, rows that
    pad a batch touch nobody's state, a one-token prompt starts from zero state, and a finished request's slot is
    used again."""
    ToyConfig = register_toys(fw)
    cfg = ToyConfig(vocab_size=101, width=40, heads=4, kv_heads=2, head_size=16, inner=56, experts=3, state_size=24,
                    decay=0.8, window=6, eps=1e-5, capturable=True)
    d = fw.root.write_random_model(tmp_path / "toy", cfg, seed=6, dtype="float32", std=0.25)
    w = P.read_weights(d, torch.float64)

    def plain_greedy(prompt, n):
        ids = list(prompt)
        for _ in range(n):
            ids.append(int(toy_plain(w, cfg, torch.tensor(ids))[-1].argmax()))
        return ids[len(prompt):]

    rng = np.random.default_rng(3)
    prompts = [[int(t) for t in rng.integers(0, 101, n)] for n in (7, 1, 12, 4, 9)]
    want = [plain_greedy(p, 14) for p in prompts]
    model = fw.root.load_model(d, "float32")
    for per_launch in (1, 4):
        e = fw.root.Engine(model, block_size=4, max_seqs=3, max_len=32, hip_graphs=True, decode_steps_per_launch=per_launch)
        assert e.runner.graphs is not None and e.runner.graphs.buckets
        reqs = [e.add_request(fw.root.Request(p, max_new_tokens=14)) for p in prompts]   # five requests, three rows
        e.run_until_idle()
        assert [r.output_ids for r in reqs] == want, per_launch
        assert any(rec.decode_batch and rec.decode_steps for rec in e.steps)


def test_rotary_part_and_block_alone(fw):
    """The rotary part against the plain rotation (a partial rotary dimension too), and the pre-norm residual
    arrangement against the plain layer, fed in two portions."""
    rt = rt_for(fw, torch.float32)
    d, nh, nkv = 32, 3, 1
    for rot in (32, 16):
        part = fw.parts.build_part("position", fw.config.PartSpec("rotary_half", "", {"head_dim": d, "rotary_dim": rot, "theta": 777.0}))
        part.load(None, rt)
        qkv = torch.randn(6, (nh + 2 * nkv) * d)

        class Ctx:
            positions = torch.tensor([0, 1, 5, 40, 41, 1000], dtype=torch.int32, device=DEV)
        dev = qkv.to(DEV)
        part.encode_and_store(dev, nh, nkv, d, Ctx, None)
        x = qkv.double().view(6, nh + 2 * nkv, d)
        cos, sin = P.rope_cos_sin(Ctx.positions.cpu(), rot, 777.0)
        want = x.clone()
        want[:, :nh + nkv, :rot] = P.apply_rope(x[:, :nh + nkv, :rot].transpose(0, 1), cos, sin).transpose(0, 1)
        torch.testing.assert_close(dev.double().cpu().view(6, nh + 2 * nkv, d), want, atol=2e-4, rtol=0)

    cfg = {"num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "rms_norm_eps": 1e-5}
    H, I, T = 64, 96, 21
    spec = fw.config.Qwen2Config(vocab_size=50, hidden_size=H, intermediate_size=I, num_hidden_layers=1, num_attention_heads=4,
                                 num_key_value_heads=2, rms_norm_eps=1e-5, rope_theta=300.0).to_spec()
    model = fw.parts.Model(spec)
    block = model.layers[0]
    t = fw.weights.random_tensors(block.tensor_specs(), 9, std=0.3, dtype="float32")
    block.load(getter(t, fw, rt), rt)
    x = torch.randn(T, H)
    w = {k: v.double() for k, v in t.items()}
    cos, sin = P.rope_cos_sin(torch.arange(T), 16, 300.0)
    want = P.decoder_layer(x.double(), w, 0, cfg, cos, sin)
    layout = fw.cache.CacheLayout(model.run_needs())
    m = fw.cache.CacheManager(layout, 4, 20, 2, 32)
    pools = fw.cache.CachePools(layout, 4, 20, 2, rt, m.max_pages_per_request)
    builder = fw.engine.BatchBuilder(m, pools, 50, rt.device)
    m.add("x")
    got, p = [], 0
    for n in (13, 8):
        m.grow("x", p + n)
        b = builder.build([fw.engine.StepEntry("x", [1] * n, [])])
        ctx = b.ctx
        xs = x[p:p + n].to(DEV).clone()
        pending = block.forward(xs, None, ctx, pools.kv_view(0, ctx.state_slots, b.slots[0]), None)
        got.append((xs if pending is None else xs + pending.float()).cpu())
        p += n
        m.advance("x", p)
    torch.testing.assert_close(torch.cat(got).double(), want, atol=2e-4, rtol=2e-4)
