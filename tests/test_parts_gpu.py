"""Each part of a layer alone against its plain formula, and the generality of
the frame: a toy architecture, defined here and registered from here, with a
mixer that keeps state of its own, a windowed attention layer with pages of its
own, a layer that runs twice and a layer that reads another call's cache; and a
second one with a feed-forward that routes tokens to experts and a position
encoding of its own.  No file of the package knows any of it."""
import json
import os
from dataclasses import dataclass

import numpy as np
import pytest
import torch

from plain import llama_plain as P
from trace_util import Trace, random_tokens, replay

from lyapunov_engine_amd.config import HF_LAYER_NAMES, HF_PREFIXES   # the toys' files use these tensor names

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ------------------------------------------------------------ parts on their own
def one_layer_core(dtype, block_size=4, **over):
    """A one-layer Llama (for its cache layout and context) with random weights."""
    from lyapunov_engine_amd.config import LlamaConfig
    from lyapunov_engine_amd.engine.core import EngineCore
    from lyapunov_engine_amd.models import build_model
    from lyapunov_engine_amd.models.llama import llama_spec
    from lyapunov_engine_amd.weights import DictSource, load_weights, random_tensors

    raw = dict(architectures=["LlamaForCausalLM"], vocab_size=100, hidden_size=80, intermediate_size=130,
               num_hidden_layers=1, num_attention_heads=5, num_key_value_heads=5, head_dim=16,
               max_position_embeddings=128, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True)
    raw.update(over)
    cfg = LlamaConfig.from_dict(raw)
    model = build_model(llama_spec(cfg))
    tensors = dict(random_tensors(model, 5, torch.float32, init_std=0.2, norm_init_std=0.2))
    tdtype = torch.float32 if dtype == "float32" else torch.bfloat16
    tensors = {k: v.to(tdtype) for k, v in tensors.items()}
    load_weights(model, DictSource(tensors), tdtype, DEV)
    core = EngineCore(model, cfg, dtype=dtype, device=DEV, num_blocks=64, block_size=block_size, num_state_slots=4)
    return core, raw, {k: v.float() for k, v in tensors.items()}


def check(got, want, dtype, what):
    """Error against the size of the result: 32-bit to 2e-5 of the largest
    value, bfloat16 (8 bits of mantissa, several roundings in a row) to 4e-2."""
    scale = float(want.abs().max())
    err = float((got.double() - want).abs().max())
    limit = (2e-5 if dtype == "float32" else 4e-2) * scale
    assert err <= limit, f"{what}: error {err:.3e} exceeds {limit:.3e} (largest value {scale:.3f})"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixer_ffn_norm_and_block_alone(dtype):
    from lyapunov_engine_amd.engine.core import StepEntry

    core, raw, w = one_layer_core(dtype)
    layer = core.model.layers[0]
    H = raw["hidden_size"]
    # two requests: a whole prompt of 11 and a second portion (positions 6..9) of another
    core.cache.add(0), core.cache.add(1)
    core.cache.extend(0, 11), core.cache.extend(1, 10)
    x_prev = torch.randn(6, H, generator=torch.Generator().manual_seed(1))
    x_new = torch.randn(11 + 4, H, generator=torch.Generator().manual_seed(2))
    tdtype = core.dtype
    # first the other request's first six tokens, through the mixer alone, to fill its pages
    ctx = core.runner.build_context([StepEntry(1, [0] * 6, 0, [])])
    caches = core.runner.layer_caches(ctx)
    layer.mixer.forward(ctx, x_prev.to(DEV, tdtype), caches[0])
    core.cache.commit(1, 6)
    ctx = core.runner.build_context([StepEntry(0, [0] * 11, 0, []), StepEntry(1, [0] * 4, 6, [])])
    caches = core.runner.layer_caches(ctx)
    xs = x_new.to(DEV, tdtype)
    inv = P.model_inv_freq(raw)
    p = "model.layers.0."

    got = layer.mixer.forward(ctx, xs, caches[0]).float().cpu()
    xa = xs[:11].float().cpu().double()
    xb = torch.cat([x_prev.to(tdtype).float(), xs[11:].float().cpu()]).double()
    wd = {k: v.double() for k, v in w.items()}
    want_a = P.attention_layer(xa, torch.arange(11), wd, p + "self_attn.", raw, inv)
    want_b = P.attention_layer(xb, torch.arange(10), wd, p + "self_attn.", raw, inv)[6:]
    check(got, torch.cat([want_a, want_b]), dtype, "mixer")

    got = layer.ffn.forward(ctx, xs).float().cpu()
    want = P.mlp(xs.float().cpu().double(), wd[p + "mlp.gate_proj.weight"], wd[p + "mlp.up_proj.weight"],
                 wd[p + "mlp.down_proj.weight"])
    check(got, want, dtype, "feed-forward")

    h = torch.randn(15, H, generator=torch.Generator().manual_seed(3)).to(DEV)
    delta = torch.randn(15, H, generator=torch.Generator().manual_seed(4)).to(DEV, tdtype)
    h0 = h.clone()
    got = layer.norm1.forward(ctx, h, delta).float().cpu()
    total = h0.cpu().double() + delta.float().cpu().double()
    torch.testing.assert_close(h.cpu().double(), total, rtol=1e-6, atol=1e-6)
    check(got, P.rms_norm(total, wd[p + "input_layernorm.weight"], raw["rms_norm_eps"]), dtype, "norm")

    # the block as a whole, on request 0 alone (fresh pages), against the plain decoder layer
    core.cache.free(0), core.cache.free(1)
    core.cache.add(2)
    core.cache.extend(2, 11)
    ctx = core.runner.build_context([StepEntry(2, [0] * 11, 0, [])])
    caches = core.runner.layer_caches(ctx)
    h = x_new[:11].to(DEV).clone()
    h2, pending = layer.forward(ctx, h, None, caches[0])
    got = h2.cpu().double() + pending.float().cpu().double()
    want = P.decoder_layer(x_new[:11].double(), torch.arange(11), wd, 0, raw, inv)
    check(got, want, dtype, "block")


def test_rotary_table_matches_the_plain_angles():
    from lyapunov_engine_amd.parts.rope import RotaryEncoding, rotary_inv_freq

    for scaling in (None, dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                               original_max_position_embeddings=64)):
        enc = RotaryEncoding(32, 500000.0, 300, scaling)
        enc.materialize(DEV, torch.float32)
        inv = P.rope_inv_freq(32, 500000.0)
        if scaling:
            inv = P.llama3_scale_inv_freq(inv, 8.0, 1.0, 4.0, 64)
        torch.testing.assert_close(rotary_inv_freq(32, 500000.0, scaling), inv, rtol=1e-6, atol=0)
        cos, sin = P.rope_cos_sin(torch.arange(300), inv)
        table = enc.table.cpu()
        assert table.shape == (300, 32)  # cosines then sines (reference: tests/test_fused_rope.py:13-24)
        torch.testing.assert_close(table[:, :16], cos[:, :16], rtol=0, atol=3e-5)
        torch.testing.assert_close(table[:, 16:], sin[:, :16], rtol=0, atol=3e-5)


# ------------------------------------------------------------- a toy architecture
TOY = dict(architectures=["ToyMixForCausalLM"], vocab_size=120, hidden_size=48, intermediate_size=72, state_size=24,
           num_heads=3, num_kv_heads=1, head_dim=16, window=6, max_position=96, eps=1e-5, theta=10000.0, decay=0.8)


@dataclass(frozen=True)
class ToyConfig:
    raw: tuple
    architectures: tuple = ("ToyMixForCausalLM",)

    @classmethod
    def from_dict(cls, d):
        return cls(tuple(sorted((k, v) for k, v in d.items() if k != "architectures" and k != "torch_dtype")),
                   tuple(d.get("architectures", cls.architectures)))

    def to_dict(self):
        return dict(self.raw, architectures=list(self.architectures))


def register_toy():
    """Everything the toy needs, through the package's public registries."""
    from lyapunov_engine_amd.config import MIXERS, LayerCall, LayerSpec, ModelSpec, PartSpec, register_architecture
    from lyapunov_engine_amd.parts import Mixer, StateSpec, WeightSource, WeightSpec

    class LinearRecurrence(Mixer):
        """s_t = decay * s_{t-1} + W_in x_t ;  y_t = W_out s_t.  The state s is
        all it keeps of a request: no pages."""

        graph_safe = False  # walks the host copy of the batch layout

        def __init__(self, hidden_size, state_size, decay):
            self.hidden_size, self.state_size, self.decay = hidden_size, state_size, decay
            self.in_proj = self.out_proj = None

        def weight_specs(self):
            return [WeightSpec("in_proj", (WeightSource("in_proj.weight", (self.state_size, self.hidden_size)),)),
                    WeightSpec("out_proj", (WeightSource("out_proj.weight", (self.hidden_size, self.state_size)),))]

        def state_spec(self):
            return StateSpec((self.state_size,), torch.float32)

        def forward(self, ctx, x, cache):
            u = x.float() @ self.in_proj.float().T
            out = torch.empty_like(u)
            for b in range(ctx.B):
                lo, hi = ctx.q_start_host[b], ctx.q_start_host[b + 1]
                slot = ctx.state_slots_host[b]
                first = ctx.ctx_len_host[b] - (hi - lo) == 0   # a new request starts from nothing
                s = torch.zeros(self.state_size, device=x.device) if first else cache.state[slot].clone()
                for t in range(lo, hi):
                    s = self.decay * s + u[t]
                    out[t] = s
                cache.state[slot] = s
            return (out @ self.out_proj.float().T).to(ctx.dtype)

    MIXERS.register("toy_linear_recurrence", LinearRecurrence, replace=True)

    def to_spec(cfg: ToyConfig) -> ModelSpec:
        c = dict(cfg.raw)
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": c["eps"]})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})
        rope = PartSpec("rope", {"dim": c["head_dim"], "theta": c["theta"], "max_position": c["max_position"]})
        attn = dict(hidden_size=H, num_heads=c["num_heads"], num_kv_heads=c["num_kv_heads"], head_dim=c["head_dim"])
        full = PartSpec("paged_attention", dict(attn, position=rope))
        windowed = PartSpec("paged_attention", dict(attn, position=None, window=c["window"]))   # no rotation either
        borrower = PartSpec("paged_attention", dict(attn, position=rope, own_kv=False))
        recur = PartSpec("toy_linear_recurrence", {"hidden_size": H, "state_size": c["state_size"],
                                                   "decay": c["decay"]})
        layers = tuple(LayerSpec("prenorm", m, ffn, norm, norm, HF_LAYER_NAMES) for m in (full, recur, windowed, borrower))
        # layer 0 runs twice (caches 0 and 3); layer 3 reads what the first call of layer 0 stored
        schedule = (LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2), LayerCall(0, 3), LayerCall(3, 0, writes=False))
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=H, layers=layers, schedule=schedule,
                         final_norm=norm, tie_word_embeddings=False, max_position=c["max_position"], **HF_PREFIXES)

    register_architecture("ToyMixForCausalLM", ToyConfig, to_spec, replace=True)


def toy_plain(folder, tokens):
    """The toy model, whole sequence, from plain parts."""
    from safetensors.torch import load_file

    c = json.load(open(os.path.join(folder, "config.json")))
    w = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    S = len(tokens)
    pos = torch.arange(S)
    nh, nkv, hd = c["num_heads"], c["num_kv_heads"], c["head_dim"]
    inv = P.rope_inv_freq(hd, c["theta"])
    cos, sin = P.rope_cos_sin(pos, inv)
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    stored = {}

    def heads(t, n):
        return t.view(S, n, hd).transpose(0, 1)

    for layer, cache, writes in ((0, 0, True), (1, 1, True), (2, 2, True), (0, 3, True), (3, 0, False)):
        p = f"model.layers.{layer}."
        x = P.rms_norm(h, w[p + "input_layernorm.weight"], c["eps"])
        if layer == 1:
            u = x @ w[p + "self_attn.in_proj.weight"].T
            s, out = torch.zeros(c["state_size"], dtype=torch.float64), []
            for t in range(S):
                s = c["decay"] * s + u[t]
                out.append(s)
            a = torch.stack(out) @ w[p + "self_attn.out_proj.weight"].T
        else:
            rotate = layer != 2
            q = heads(x @ w[p + "self_attn.q_proj.weight"].T, nh)
            q = P.apply_rope(q, cos, sin) if rotate else q
            if writes:
                k = heads(x @ w[p + "self_attn.k_proj.weight"].T, nkv)
                k = P.apply_rope(k, cos, sin) if rotate else k
                stored[cache] = (k, heads(x @ w[p + "self_attn.v_proj.weight"].T, nkv))
            k, v = stored[cache]
            o = P.attention(q, k, v, pos, pos, window=c["window"] if layer == 2 else 0)
            a = o.transpose(0, 1).reshape(S, nh * hd) @ w[p + "self_attn.o_proj.weight"].T
        h = h + a
        x = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], c["eps"])
        h = h + P.mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["lm_head.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype):
    from lyapunov_engine_amd.config import ARCHITECTURES, MIXERS
    from lyapunov_engine_amd.models import build_model
    from lyapunov_engine_amd.weights import write_random_model

    register_toy()
    try:
        folder = str(tmp_path / "toy")
        write_random_model(dict(TOY), folder, seed=1, dtype=dtype, init_std=0.15, norm_init_std=0.1)
        arch = ARCHITECTURES.get("ToyMixForCausalLM")
        model = build_model(arch.to_spec(arch.config_class.from_dict(TOY)))
        layout = model.cache_layout()
        assert len(layout.groups) == 2                       # all keys, and a window of them: pages of their own
        assert layout.groups[0].buffers == (0, 3) and layout.groups[1].buffers == (2,)
        assert layout.groups[1].spec.window == 6 and list(layout.states) == [1]
        names = model.expected_tensors()
        assert "model.layers.1.self_attn.in_proj.weight" in names
        assert "model.layers.3.self_attn.k_proj.weight" not in names   # the borrower has no keys of its own

        reqs = {"x": random_tokens(60, 120, seed=2), "y": random_tokens(23, 120, seed=3),
                "z": random_tokens(41, 120, seed=4)}
        want = {k: toy_plain(folder, v) for k, v in reqs.items()}
        from trace_util import compare

        whole = Trace(reqs)
        for rid in reqs:
            whole.step([(rid, len(reqs[rid]))], end=[rid])
        compare(whole, replay(folder, dtype, whole), want, dtype, "toy whole")

        cut = Trace(reqs)
        cut.step([("x", 7), ("y", 23)], end=["y"])
        cut.step([("x", 2), ("z", 30)])
        for _ in range(9):
            cut.step([("x", 1), ("z", 1)])
        cut.step([("x", 42), ("z", 2)], end=["x", "z"])
        compare(cut, replay(folder, dtype, cut), want, dtype, "toy cut")
        # the windowed layers' group with a pool of its own size and smaller pages: a window of 6 keys needs
        # few pages per request beside those of the portion a step brings (here up to 42 tokens)
        got = replay(folder, dtype, cut, cache_groups=[None, (24, 4)])
        compare(cut, got, want, dtype, "toy cut, pools of two sizes")
        with pytest.raises(ValueError, match="cache_groups names 3 groups"):
            replay(folder, dtype, cut, cache_groups=[None, None, (8, 8)])

        # through the generating engine: greedy tokens are the plain model's; with a state that a step
        # changes in place no step is started ahead (one that had to be dropped could not be run again)
        import lyapunov_engine_amd as L
        llm = L.LLM(folder, dtype=dtype, num_blocks=64, block_size=4, max_num_seqs=4)
        assert llm.engine._look_ahead is False
        prompt = reqs["y"][:9]
        got = llm.generate([prompt], L.SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))[0].output_tokens
        toks = list(prompt)
        for i in range(6):
            logits = toy_plain(folder, toks)[-1]
            top = torch.topk(logits, 2).values
            if got[i] != int(logits.argmax()):
                assert dtype == "bfloat16" and float(top[0] - top[1]) < 0.25, (i, got)
                break
            toks.append(got[i])
    finally:
        ARCHITECTURES.unregister("ToyMixForCausalLM")
        MIXERS.unregister("toy_linear_recurrence")


# ------------------------------------------- a second toy: routing, other positions
TOY2 = dict(architectures=["ToyRoutedForCausalLM"], vocab_size=90, hidden_size=64, num_heads=2, num_kv_heads=1,
            head_dim=32, rotary_dim=16, experts=3, expert_size=48, intermediate_size=80, max_position=128, eps=1e-6,
            slope=0.37)


def register_toy2():
    """A feed-forward that routes every token to one of several experts, and a
    position encoding that is neither the package's rope nor its "none": both
    defined here and registered from here."""
    from lyapunov_engine_amd.config import (FEED_FORWARDS, POSITION_ENCODINGS, LayerSpec, ModelSpec, PartSpec,
                                            default_schedule, register_architecture)
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts import FeedForward, PositionEncoding, WeightSource, WeightSpec

    class RoutedExperts(FeedForward):
        """Router logits in 32-bit; a token goes to its best expert alone and its
        output is weighted by that expert's softmax probability."""

        graph_safe = False   # which rows go where is read on the host

        def __init__(self, hidden_size, expert_size, experts):
            self.hidden_size, self.expert_size, self.experts = hidden_size, expert_size, experts
            self.router = None

        def weight_specs(self):
            E, H = self.expert_size, self.hidden_size
            specs = [WeightSpec("router", (WeightSource("router.weight", (self.experts, H)),))]
            for e in range(self.experts):
                specs.append(WeightSpec(f"gate_up_{e}", (WeightSource(f"experts.{e}.gate_proj.weight", (E, H)),
                                                         WeightSource(f"experts.{e}.up_proj.weight", (E, H)))))
                specs.append(WeightSpec(f"down_{e}", (WeightSource(f"experts.{e}.down_proj.weight", (H, E)),)))
            return specs

        def forward(self, ctx, x):
            logits = ops.linear(x, self.router, out_dtype=torch.float32)
            prob, choice = torch.softmax(logits, dim=-1).max(dim=-1)
            out = torch.zeros((x.shape[0], self.hidden_size), dtype=torch.float32, device=x.device)
            for e in range(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    act = ops.linear_swiglu(x[rows].contiguous(), getattr(self, f"gate_up_{e}"), 0)
                    y = ops.linear(act, getattr(self, f"down_{e}"), out_dtype=torch.float32)
                    out[rows] = y * prob[rows, None]
            return out.to(ctx.dtype)

    class LinearAngles(PositionEncoding):
        """Rotates the first `dim` features of a head by angles pos * slope / (i + 1)."""

        def __init__(self, dim, slope, max_position):
            self.rotary_dim, self.slope, self.max_position = dim, slope, max_position
            self.table = None

        def materialize(self, device, dtype):
            freq = self.slope / torch.arange(1, self.rotary_dim // 2 + 1, dtype=torch.float32)
            angles = torch.outer(torch.arange(self.max_position, dtype=torch.float32), freq)
            self.table = torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous().to(device)

    FEED_FORWARDS.register("toy_routed_experts", RoutedExperts, replace=True)
    POSITION_ENCODINGS.register("toy_linear_angles", LinearAngles, replace=True)

    def to_spec(cfg: ToyConfig) -> ModelSpec:
        c = dict(cfg.raw)
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": c["eps"]})
        pos = PartSpec("toy_linear_angles", {"dim": c["rotary_dim"], "slope": c["slope"],
                                             "max_position": c["max_position"]})
        attn = PartSpec("paged_attention", dict(hidden_size=H, num_heads=c["num_heads"],
                                                num_kv_heads=c["num_kv_heads"], head_dim=c["head_dim"], position=pos))
        routed = PartSpec("toy_routed_experts", {"hidden_size": H, "expert_size": c["expert_size"],
                                                 "experts": c["experts"]})
        dense = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})
        layers = (LayerSpec("prenorm", attn, routed, norm, norm, HF_LAYER_NAMES),
                  LayerSpec("prenorm", attn, dense, norm, norm, HF_LAYER_NAMES))
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=H, layers=layers, schedule=default_schedule(2),
                         final_norm=norm, tie_word_embeddings=True, max_position=c["max_position"], **HF_PREFIXES)

    register_architecture("ToyRoutedForCausalLM", ToyConfig, to_spec, replace=True)


def toy2_plain(folder, tokens):
    from safetensors.torch import load_file

    c = json.load(open(os.path.join(folder, "config.json")))
    w = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    S, nh, nkv, hd, rot = len(tokens), c["num_heads"], c["num_kv_heads"], c["head_dim"], c["rotary_dim"]
    pos = torch.arange(S)
    freq = (c["slope"] / torch.arange(1, rot // 2 + 1, dtype=torch.float32)).double()
    angles = torch.outer(pos.double(), freq)
    cos, sin = torch.cat((angles.cos(), angles.cos()), -1), torch.cat((angles.sin(), angles.sin()), -1)

    def rotate(t):   # the first `rot` features of every head, the rest as they are
        return torch.cat((P.apply_rope(t[..., :rot], cos, sin), t[..., rot:]), dim=-1)

    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    for layer in range(2):
        p = f"model.layers.{layer}."
        x = P.rms_norm(h, w[p + "input_layernorm.weight"], c["eps"])
        q = rotate((x @ w[p + "self_attn.q_proj.weight"].T).view(S, nh, hd).transpose(0, 1))
        k = rotate((x @ w[p + "self_attn.k_proj.weight"].T).view(S, nkv, hd).transpose(0, 1))
        v = (x @ w[p + "self_attn.v_proj.weight"].T).view(S, nkv, hd).transpose(0, 1)
        o = P.attention(q, k, v, pos, pos)
        h = h + o.transpose(0, 1).reshape(S, nh * hd) @ w[p + "self_attn.o_proj.weight"].T
        x = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], c["eps"])
        if layer == 0:
            prob, choice = torch.softmax(x @ w[p + "mlp.router.weight"].T, dim=-1).max(dim=-1)
            y = torch.zeros_like(h)
            for t in range(S):
                e = int(choice[t])
                m = f"{p}mlp.experts.{e}."
                y[t] = prob[t] * P.mlp(x[t:t + 1], w[m + "gate_proj.weight"], w[m + "up_proj.weight"],
                                       w[m + "down_proj.weight"])[0]
            h = h + y
        else:
            h = h + P.mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_routed_feed_forward_and_another_position_encoding(tmp_path, dtype):
    from lyapunov_engine_amd.config import ARCHITECTURES, FEED_FORWARDS, POSITION_ENCODINGS
    from lyapunov_engine_amd.weights import write_random_model
    from trace_util import compare

    register_toy2()
    try:
        folder = str(tmp_path / "toy2")
        # With this seed every token's best expert leads the second by 0.13 or more (logits up to
        # 4.4) and every expert gets tokens: near a tie the engine and the plain model, which round
        # differently, would send a token to different experts, which is no fault of either.
        write_random_model(dict(TOY2), folder, seed=138, dtype=dtype, init_std=0.15, norm_init_std=0.1)
        reqs = {"x": random_tokens(50, 90, seed=5), "y": random_tokens(19, 90, seed=6)}
        want = {k: toy2_plain(folder, v) for k, v in reqs.items()}
        whole = Trace(reqs)
        for rid in reqs:
            whole.step([(rid, len(reqs[rid]))], end=[rid])
        compare(whole, replay(folder, dtype, whole), want, dtype, "routed whole")
        cut = Trace(reqs)
        cut.step([("x", 11), ("y", 3)])
        cut.step([("x", 2), ("y", 16)], end=["y"])
        for _ in range(12):
            cut.step([("x", 1)])
        cut.step([("x", 25)], end=["x"])
        compare(cut, replay(folder, dtype, cut), want, dtype, "routed cut")
    finally:
        ARCHITECTURES.unregister("ToyRoutedForCausalLM")
        FEED_FORWARDS.unregister("toy_routed_experts")
        POSITION_ENCODINGS.unregister("toy_linear_angles")


# ----------------------- a third toy: a mixer with state, lists of its own, and graphs
TOY3 = dict(architectures=["ToyScanForCausalLM"], vocab_size=100, hidden_size=64, intermediate_size=96, state_size=32,
            num_heads=2, num_kv_heads=1, head_dim=32, max_position=200, eps=1e-5, theta=10000.0, decay=0.7)


def register_toy3():
    """A recurrence that never looks at the host's copy of the batch: what it needs to know about
    the step's requests it asks for through a planner of its own, as device lists, and so its
    decode steps can be recorded once and replayed."""
    from lyapunov_engine_amd.config import MIXERS, LayerSpec, ModelSpec, PartSpec, default_schedule, register_architecture
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts import Mixer, StateSpec, StepPlanner, WeightSource, WeightSpec

    class Segments(StepPlanner):
        """Per request: 1 if it starts from nothing.  meta: the most tokens any request brings
        (the number of rounds the scan takes; in a recorded step the most it could bring)."""
        key = ("toy_segments",)

        def plan(self, batch):
            fresh = (batch.ctx_len - batch.count == 0).astype(np.int32)
            longest = int(batch.count.max()) if batch.fixed is None else (batch.fixed.tokens or 1)
            return {"fresh": fresh}, {"longest": longest}

    class ScanOnDevice(Mixer):
        """s_t = decay * s_{t-1} + W_in x_t ;  y_t = W_out s_t, one round per token position within
        the requests, all requests at once."""

        def __init__(self, hidden_size, state_size, decay):
            self.hidden_size, self.state_size, self.decay = hidden_size, state_size, decay
            self.in_proj = self.out_proj = None

        def weight_specs(self):
            return [WeightSpec("in_proj", (WeightSource("in_proj.weight", (self.state_size, self.hidden_size)),)),
                    WeightSpec("out_proj", (WeightSource("out_proj.weight", (self.hidden_size, self.state_size)),))]

        def state_spec(self):
            return StateSpec((self.state_size,), torch.float32)

        def step_planner(self):
            return Segments()

        def forward(self, ctx, x, cache):
            plan = ctx.plans[Segments.key]
            u = ops.linear(x, self.in_proj, out_dtype=torch.float32)                  # [T, S]
            slots = ctx.state_slots.long()
            first = ctx.q_start[:-1].long()
            count = (ctx.q_start[1:] - ctx.q_start[:-1]).long()
            keep = (1 - plan.arrays["fresh"]).float()[:, None]
            s = cache.state.index_select(0, slots) * keep                               # [B, S]
            out = torch.zeros((ctx.T + 1, self.state_size), dtype=torch.float32, device=x.device)
            for j in range(plan.meta["longest"]):
                live = (count > j)
                at = torch.where(live, first + j, torch.full_like(first, ctx.T))       # done requests write row T
                s = torch.where(live[:, None], self.decay * s + u.index_select(0, at.clamp(max=ctx.T - 1)), s)
                out.index_copy_(0, at, s)
            cache.state.index_copy_(0, slots, s)      # padded rows all write the spare slot
            return ops.linear(ops.cast(out[:ctx.T].contiguous(), ctx.dtype), self.out_proj, out_dtype=ctx.dtype)

    MIXERS.register("toy_scan_on_device", ScanOnDevice, replace=True)

    def to_spec(cfg: ToyConfig) -> ModelSpec:
        c = dict(cfg.raw)
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": c["eps"]})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})
        rope = PartSpec("rope", {"dim": c["head_dim"], "theta": c["theta"], "max_position": c["max_position"]})
        attn = PartSpec("paged_attention", dict(hidden_size=H, num_heads=c["num_heads"], num_kv_heads=c["num_kv_heads"],
                                                head_dim=c["head_dim"], position=rope))
        scan = PartSpec("toy_scan_on_device", {"hidden_size": H, "state_size": c["state_size"], "decay": c["decay"]})
        layers = (LayerSpec("prenorm", attn, ffn, norm, norm, HF_LAYER_NAMES),
                  LayerSpec("prenorm", scan, ffn, norm, norm, HF_LAYER_NAMES))
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=H, layers=layers, schedule=default_schedule(2),
                         final_norm=norm, tie_word_embeddings=True, max_position=c["max_position"], **HF_PREFIXES)

    register_architecture("ToyScanForCausalLM", ToyConfig, to_spec, replace=True)


def toy3_plain(folder, tokens):
    from safetensors.torch import load_file

    c = json.load(open(os.path.join(folder, "config.json")))
    w = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    S, nh, nkv, hd = len(tokens), c["num_heads"], c["num_kv_heads"], c["head_dim"]
    pos = torch.arange(S)
    cos, sin = P.rope_cos_sin(pos, P.rope_inv_freq(hd, c["theta"]))
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    for layer in range(2):
        p = f"model.layers.{layer}."
        x = P.rms_norm(h, w[p + "input_layernorm.weight"], c["eps"])
        if layer == 0:
            q = P.apply_rope((x @ w[p + "self_attn.q_proj.weight"].T).view(S, nh, hd).transpose(0, 1), cos, sin)
            k = P.apply_rope((x @ w[p + "self_attn.k_proj.weight"].T).view(S, nkv, hd).transpose(0, 1), cos, sin)
            v = (x @ w[p + "self_attn.v_proj.weight"].T).view(S, nkv, hd).transpose(0, 1)
            a = P.attention(q, k, v, pos, pos).transpose(0, 1).reshape(S, nh * hd) @ w[p + "self_attn.o_proj.weight"].T
        else:
            u = x @ w[p + "self_attn.in_proj.weight"].T
            s, out = torch.zeros(c["state_size"], dtype=torch.float64), []
            for t in range(S):
                s = c["decay"] * s + u[t]
                out.append(s)
            a = torch.stack(out) @ w[p + "self_attn.out_proj.weight"].T
        h = h + a
        x = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], c["eps"])
        h = h + P.mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_stateful_mixer_with_lists_of_its_own_decodes_through_graphs(tmp_path, dtype):
    """Registered from here, with a planner of its own: the step function uploads its list with the
    step's tables, the recorded decode step replays with it, padded rows touch no request's state.
    Replay against the plain model; generation with graphs against generation without (three
    requests that start and end at different steps, so the batch and its padding change while the
    graphs are replayed), and in 32-bit against the plain model's greedy tokens."""
    import lyapunov_engine_amd as L
    from lyapunov_engine_amd.config import ARCHITECTURES, MIXERS
    from lyapunov_engine_amd.weights import write_random_model
    from trace_util import compare

    register_toy3()
    try:
        folder = str(tmp_path / "toy3")
        write_random_model(dict(TOY3), folder, seed=4, dtype=dtype, init_std=0.15, norm_init_std=0.1)
        reqs = {"x": random_tokens(45, 100, seed=7), "y": random_tokens(18, 100, seed=8)}
        want = {k: toy3_plain(folder, v) for k, v in reqs.items()}
        cut = Trace(reqs)
        cut.step([("x", 9), ("y", 3)])
        cut.step([("x", 2), ("y", 15)], end=["y"])
        for _ in range(10):
            cut.step([("x", 1)])
        cut.step([("x", 24)], end=["x"])
        compare(cut, replay(folder, dtype, cut), want, dtype, "scan cut")

        prompts = [reqs["x"][:12], reqs["y"][:5], reqs["x"][20:27]]
        lengths = [30, 12, 21]

        def run(graphs):
            llm = L.LLM(folder, dtype=dtype, num_blocks=64, block_size=4, max_num_seqs=4, enable_graphs=graphs)
            params = [L.SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True) for n in lengths]
            outs = llm.generate(prompts, params)
            return [o.output_tokens for o in outs], llm.engine

        with_graphs, engine = run(True)
        assert engine.graphs.safe and engine.graphs.captured, "the toy's decode steps were meant to be recorded"
        assert {key[0] for key in engine.graphs.captured} >= {1, 2, 3}       # batches of 3, 2 and 1 as requests end
        eager, _ = run(False)
        assert with_graphs == eager
        if dtype == "float32":
            toks = list(prompts[0])
            for t in with_graphs[0]:
                assert t == int(toy3_plain(folder, toks)[-1].argmax())
                toks.append(t)
        # a short prompt alone in its step is a recorded step too (16 token rows, of which 12 are live)
        llm = L.LLM(folder, dtype=dtype, num_blocks=64, block_size=4, max_num_seqs=4)
        one = llm.generate([prompts[0]], L.SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))[0].output_tokens
        assert any(len(key) == 3 for key in llm.engine.graphs.captured)
        assert one == with_graphs[0][:8]
    finally:
        ARCHITECTURES.unregister("ToyScanForCausalLM")
        MIXERS.unregister("toy_scan_on_device")


# ----------------------- a fourth toy: other ends (a scaled embedding, capped logits), four norms a layer
TOY4 = dict(architectures=["ToyEndsForCausalLM"], vocab_size=130, hidden_size=64, intermediate_size=112,
            num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16, max_position_embeddings=160,
            rms_norm_eps=1e-5, rope_theta=10000.0, embed_scale=8.0, logit_cap=2.0)


def register_toy4():
    """An embedding that scales its rows, an output head that caps its logits and has a bias of
    its own, and an arrangement of a layer with a norm after each branch as well as before it: all
    defined and registered here; mixer, feed-forward and norms are the package's."""
    from lyapunov_engine_amd.config import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, LayerSpec, ModelSpec,
                                            PartSpec, default_schedule, register_architecture)
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts import Block, Embedding, Head, WeightSource, WeightSpec

    class Sandwich(Block):
        """h += post1(mixer(norm1(h))); h += post2(ffn(norm2(h))).  The two further norms come
        from LayerSpec.extra."""

        def __init__(self, spec):
            self.norm1, self.norm2 = NORMS.build(spec.norm1), NORMS.build(spec.norm2)
            self.post1, self.post2 = NORMS.build(spec.extra["post_mixer"]), NORMS.build(spec.extra["post_ffn"])
            self.mixer, self.ffn = MIXERS.build(spec.mixer), FEED_FORWARDS.build(spec.ffn)

        def children(self):
            return {"input_layernorm.": self.norm1, "self_attn.": self.mixer, "post_mixer_norm.": self.post1,
                    "post_attention_layernorm.": self.norm2, "mlp.": self.ffn, "post_ffn_norm.": self.post2}

        def branch(self, ctx, norm, part, post, h, delta, *cache):
            x = norm.forward(ctx, h, ops.as_delta(delta, ctx.dtype))
            y = ops.as_delta(part.forward(ctx, x, *cache), torch.float32)       # the branch's output, summed up
            return post.forward(ctx, y)

        def forward(self, ctx, h, delta, cache):
            a = self.branch(ctx, self.norm1, self.mixer, self.post1, h, delta, cache)
            return h, self.branch(ctx, self.norm2, self.ffn, self.post2, h, a)

    BLOCKS.register("toy_sandwich", Sandwich, replace=True)

    class ScaledLookup(Embedding):
        def __init__(self, vocab_size, hidden_size, scale):
            self.vocab_size, self.hidden_size, self.scale = vocab_size, hidden_size, scale
            self.weight = None

        def weight_specs(self):
            return [WeightSpec("weight", (WeightSource("weight", (self.vocab_size, self.hidden_size)),))]

        def forward(self, ctx, token_ids):
            h = torch.empty((token_ids.numel(), self.hidden_size), dtype=torch.float32, device=ctx.device)
            return ops.embedding(token_ids, self.weight, h).mul_(self.scale)

    class CappedHead(Head):
        """cap * tanh((x W^T + b) / cap): the embedding's matrix, a bias of its own."""

        def __init__(self, vocab_size, hidden_size, cap):
            self.vocab_size, self.hidden_size, self.cap = vocab_size, hidden_size, cap
            self.bias, self.table = None, None

        def tie(self, embedding):
            self.table = embedding

        def weight_specs(self):
            return [WeightSpec("bias", (WeightSource("bias", (self.vocab_size,)),))]

        def forward(self, ctx, x):
            # the product's row maxima do not hold for capped, biased logits: only the values are returned
            logits = ops.lm_head(x, self.table.weight)[0] + self.bias.float()
            return torch.tanh(logits / self.cap) * self.cap

    EMBEDDINGS.register("toy_scaled_lookup", ScaledLookup, replace=True)
    HEADS.register("toy_capped_head", CappedHead, replace=True)

    def to_spec(cfg: ToyConfig) -> ModelSpec:
        c = dict(cfg.raw)
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": c["rms_norm_eps"]})
        pos = PartSpec("rope", {"dim": c["head_dim"], "theta": c["rope_theta"], "max_position": c["max_position_embeddings"],
                                "scaling": None})
        attn = PartSpec("paged_attention", dict(hidden_size=H, num_heads=c["num_attention_heads"],
                                                num_kv_heads=c["num_key_value_heads"], head_dim=c["head_dim"], position=pos))
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})
        n = c["num_hidden_layers"]
        layer = LayerSpec("toy_sandwich", attn, ffn, norm, norm, HF_LAYER_NAMES, extra={"post_mixer": norm, "post_ffn": norm})
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=H, layers=tuple(layer for _ in range(n)),
                         schedule=default_schedule(n), final_norm=norm, tie_word_embeddings=True,
                         max_position=c["max_position_embeddings"],
                         embedding=PartSpec("toy_scaled_lookup", {"scale": c["embed_scale"]}),
                         head=PartSpec("toy_capped_head", {"cap": c["logit_cap"]}), **HF_PREFIXES)

    register_architecture("ToyEndsForCausalLM", ToyConfig, to_spec, replace=True)


def toy4_plain(folder, tokens):
    from safetensors.torch import load_file

    c = json.load(open(os.path.join(folder, "config.json")))
    w = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    positions = torch.arange(len(tokens))
    inv_freq = P.model_inv_freq(c)
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)] * c["embed_scale"]
    eps = c["rms_norm_eps"]
    for i in range(c["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = P.attention_layer(P.rms_norm(h, w[p + "input_layernorm.weight"], eps), positions, w, p + "self_attn.", c, inv_freq)
        h = h + P.rms_norm(a, w[p + "post_mixer_norm.weight"], eps)
        m = P.mlp(P.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps), w[p + "mlp.gate_proj.weight"],
                  w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        h = h + P.rms_norm(m, w[p + "post_ffn_norm.weight"], eps)
    logits = P.rms_norm(h, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T + w["lm_head.bias"]
    return torch.tanh(logits / c["logit_cap"]) * c["logit_cap"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_another_embedding_and_another_output_head(tmp_path, dtype):
    """The model's two ends are parts like the others: an architecture names an embedding and a
    head of its own, with their own tensors and constants, and an arrangement of a layer with more
    parts than the usual four, and nothing in the package changes.  Whole prompts, portions
    beside decoded tokens, and recorded decode steps through the engine."""
    import lyapunov_engine_amd as L
    from lyapunov_engine_amd.config import ARCHITECTURES, BLOCKS, EMBEDDINGS, HEADS
    from lyapunov_engine_amd.weights import write_random_model
    from trace_util import compare

    register_toy4()
    try:
        folder = str(tmp_path / "toy4")
        write_random_model(dict(TOY4), folder, seed=9, dtype=dtype, init_std=0.08, norm_init_std=0.1)
        from safetensors.torch import load_file
        names = set(load_file(os.path.join(folder, "model.safetensors")))
        assert "lm_head.bias" in names and "lm_head.weight" not in names and "model.layers.1.post_ffn_norm.weight" in names
        reqs = {"x": random_tokens(60, 130, seed=15), "y": random_tokens(23, 130, seed=16)}
        want = {k: toy4_plain(folder, v) for k, v in reqs.items()}
        assert float(want["x"].abs().max()) > 0.8 * TOY4["logit_cap"]        # the cap is felt
        whole = Trace(reqs)
        for rid in reqs:
            whole.step([(rid, len(reqs[rid]))], end=[rid])
        compare(whole, replay(folder, dtype, whole), want, dtype, "ends whole")
        cut = Trace(reqs)
        cut.step([("x", 13), ("y", 4)])
        cut.step([("x", 2), ("y", 19)], end=["y"])
        for _ in range(10):
            cut.step([("x", 1)])
        cut.step([("x", 35)], end=["x"])
        compare(cut, replay(folder, dtype, cut), want, dtype, "ends cut")
        # through the engine, decode steps recorded: greedy tokens against the plain model's
        llm = L.LLM(folder, dtype=dtype, num_blocks=32, block_size=16, enable_graphs=True, warmup=False)
        assert llm.engine.graphs is not None and llm.engine.graphs.safe
        prompt = reqs["y"]
        got = llm.generate([prompt], L.SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True))[0].output_tokens
        toks = list(prompt)
        for i in range(6):
            logits = toy4_plain(folder, toks)[-1]
            top = torch.topk(logits, 2).values
            if got[i] != int(logits.argmax()):
                assert dtype == "bfloat16" and float(top[0] - top[1]) < 0.25, (i, got)
                break
            toks.append(got[i])
    finally:
        ARCHITECTURES.unregister("ToyEndsForCausalLM")
        EMBEDDINGS.unregister("toy_scaled_lookup")
        HEADS.unregister("toy_capped_head")
        BLOCKS.unregister("toy_sandwich")


# --------------------------------- a fifth toy: a mixer with a page layout of its own
TOY5 = dict(architectures=["ToyLatentForCausalLM"], vocab_size=110, hidden_size=64, intermediate_size=96, latent=24,
            num_heads=2, num_kv_heads=2, head_dim=16, max_position=128, eps=1e-5, theta=10000.0)


def register_toy5():
    """A mixer that keeps one vector per token in pages (no separate values, kept in 32-bit whatever
    the engine's precision), in a layout that is its own: what a page holds is said by the mixer's
    ``PagedSpec`` and nowhere else."""
    from lyapunov_engine_amd.config import MIXERS, LayerSpec, ModelSpec, PartSpec, default_schedule, register_architecture
    from lyapunov_engine_amd.parts import SLOT, Mixer, PagedSpec, PageTensor, WeightSource, WeightSpec

    class LatentAttention(Mixer):
        """c_t = W_c x_t is all a token leaves behind; token t reads softmax_s<=t(q_t . c_s / sqrt(L)) c_s."""

        graph_safe = False   # walks the host copy of the batch layout

        def __init__(self, hidden_size, latent):
            self.hidden_size, self.latent = hidden_size, latent
            self.q_proj = self.c_proj = self.o_proj = None

        def weight_specs(self):
            return [WeightSpec("q_proj", (WeightSource("q_proj.weight", (self.latent, self.hidden_size)),)),
                    WeightSpec("c_proj", (WeightSource("c_proj.weight", (self.latent, self.hidden_size)),)),
                    WeightSpec("o_proj", (WeightSource("o_proj.weight", (self.hidden_size, self.latent)),))]

        def cache_spec(self):
            return PagedSpec((PageTensor("latent", (SLOT, self.latent), torch.float32),))

        def forward(self, ctx, x, cache):
            assert set(cache.pages) == {"latent"} and cache.k is None and cache.v is None
            pool = cache.pages["latent"]                      # [pages, page size, latent], float32
            assert pool.dtype == torch.float32 and pool.shape[1:] == (cache.group.page_size, self.latent)
            flat = pool.view(-1, self.latent)
            xf = x.float()
            q, c = xf @ self.q_proj.float().T, xf @ self.c_proj.float().T
            flat[cache.group.slot_mapping.long()] = c
            out = torch.empty_like(q)
            ps = cache.group.page_size
            for b in range(ctx.B):
                lo, hi, n = ctx.q_start_host[b], ctx.q_start_host[b + 1], ctx.ctx_len_host[b]
                pages = cache.group.block_tables[b, :-(-n // ps)].long()
                slots = (pages[:, None] * ps + torch.arange(ps, device=x.device)[None, :]).reshape(-1)[:n]
                keys = flat[slots]                                            # [n, latent]
                scores = q[lo:hi] @ keys.T / self.latent ** 0.5
                pos = torch.arange(n - (hi - lo), n, device=x.device)
                scores = scores.masked_fill(torch.arange(n, device=x.device)[None, :] > pos[:, None], float("-inf"))
                out[lo:hi] = torch.softmax(scores, dim=-1) @ keys
            return (out @ self.o_proj.float().T).to(ctx.dtype)

    MIXERS.register("toy_latent_attention", LatentAttention, replace=True)

    def to_spec(cfg: ToyConfig) -> ModelSpec:
        c = dict(cfg.raw)
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": c["eps"]})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})
        rope = PartSpec("rope", {"dim": c["head_dim"], "theta": c["theta"], "max_position": c["max_position"]})
        attn = PartSpec("paged_attention", dict(hidden_size=H, num_heads=c["num_heads"], num_kv_heads=c["num_kv_heads"],
                                                head_dim=c["head_dim"], position=rope))
        latent = PartSpec("toy_latent_attention", {"hidden_size": H, "latent": c["latent"]})
        layers = (LayerSpec("prenorm", latent, ffn, norm, norm, HF_LAYER_NAMES),
                  LayerSpec("prenorm", attn, ffn, norm, norm, HF_LAYER_NAMES))
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=H, layers=layers, schedule=default_schedule(2),
                         final_norm=norm, tie_word_embeddings=True, max_position=c["max_position"], **HF_PREFIXES)

    register_architecture("ToyLatentForCausalLM", ToyConfig, to_spec, replace=True)


def toy5_plain(folder, tokens):
    from safetensors.torch import load_file

    c = json.load(open(os.path.join(folder, "config.json")))
    w = {k: v.double() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    S = len(tokens)
    pos = torch.arange(S)
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    # layer 0: the latent mixer
    p = "model.layers.0."
    x = P.rms_norm(h, w[p + "input_layernorm.weight"], c["eps"])
    q, lat = x @ w[p + "self_attn.q_proj.weight"].T, x @ w[p + "self_attn.c_proj.weight"].T
    scores = (q @ lat.T / c["latent"] ** 0.5).masked_fill(pos[None, :] > pos[:, None], float("-inf"))
    h = h + (torch.softmax(scores, dim=-1) @ lat) @ w[p + "self_attn.o_proj.weight"].T
    x = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], c["eps"])
    h = h + P.mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    # layer 1: the package's attention
    raw = dict(num_attention_heads=c["num_heads"], num_key_value_heads=c["num_kv_heads"], head_dim=c["head_dim"],
               rms_norm_eps=c["eps"])
    inv = P.rope_inv_freq(c["head_dim"], c["theta"])
    h = P.decoder_layer(h, pos, w, 1, raw, inv)
    return P.rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_with_a_page_layout_of_its_own(tmp_path, dtype):
    """The pages' layout belongs to the mixer: a mixer registered from here keeps one 32-bit vector
    per token (no values), gets a pool of exactly that shape and type beside the attention layer's
    key and value pools, and the cache manager, the step function and the replay run it, pages
    given back and used again, without a change to the package."""
    from lyapunov_engine_amd.config import ARCHITECTURES, MIXERS
    from lyapunov_engine_amd.engine.core import EngineCore
    from lyapunov_engine_amd.weights import write_random_model
    from trace_util import compare

    register_toy5()
    try:
        folder = str(tmp_path / "toy5")
        write_random_model(dict(TOY5), folder, seed=21, dtype=dtype, init_std=0.15, norm_init_std=0.1)
        core = EngineCore.from_folder(folder, dtype=dtype, num_blocks=8, block_size=4, num_state_slots=2)
        layout = core.model.cache_layout()
        assert len(layout.groups) == 2 and [t.name for t in layout.groups[0].spec.tensors] == ["latent"]
        assert [t.name for t in layout.groups[1].spec.tensors] == ["k", "v"]
        assert {n: (tuple(t.shape), t.dtype) for n, t in core.pools.paged[0].items()} == \
            {"latent": ((1, 8, 4, TOY5["latent"]), torch.float32)}
        assert core.pools.paged[1]["v"].shape == (1, 8, TOY5["num_kv_heads"], TOY5["head_dim"], 4)
        del core
        reqs = {"x": random_tokens(50, 110, seed=22), "y": random_tokens(19, 110, seed=23), "z": random_tokens(30, 110, seed=24)}
        want = {k: toy5_plain(folder, v) for k, v in reqs.items()}
        whole = Trace(reqs)
        for rid in reqs:
            whole.step([(rid, len(reqs[rid]))], end=[rid])
        compare(whole, replay(folder, dtype, whole), want, dtype, "latent whole")
        cut = Trace(reqs)
        cut.step([("x", 9), ("y", 19)], end=["y"])
        cut.step([("x", 3), ("z", 17)])
        for _ in range(8):
            cut.step([("x", 1), ("z", 1)])
        cut.step([("x", 30), ("z", 5)], end=["x", "z"])
        compare(cut, replay(folder, dtype, cut), want, dtype, "latent cut")
    finally:
        ARCHITECTURES.unregister("ToyLatentForCausalLM")
        MIXERS.unregister("toy_latent_attention")
