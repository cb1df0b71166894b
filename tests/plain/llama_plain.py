"""A plain, slow Llama in torch on the CPU: whole sequences, no cache, one
function per part.  It is what the engine is compared with, and it shares no
code with the engine (it imports nothing from the package; the model folder is
read with the safetensors library).

Each function cites the place in the reference it is written from
(/root/reference, read, never run).  Where the reference has nothing (llama3
frequency scaling, tied head, a window) the docstring says where the formula
comes from instead.
"""
from __future__ import annotations

import json
import math
import os

import torch


# ----------------------------------------------------------------------- parts
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """python/lyapunov_engine/ops.py:49-50:
    variance = x.pow(2).mean(-1, keepdim=True); out = x * rsqrt(variance + eps) * weight."""
    variance = x.pow(2).mean(-1, keepdim=True)
    return x * torch.rsqrt(variance + eps) * weight


def rope_inv_freq(dim: int, theta: float) -> torch.Tensor:
    """python/lyapunov_engine/models/llama.py:180-184:
    inv_freq = 1.0 / (theta ** (arange(0, dim, 2).float() / dim)), in 32-bit."""
    return 1.0 / (theta ** (torch.arange(0, dim, 2).float() / dim))


def llama3_scale_inv_freq(inv_freq: torch.Tensor, factor: float, low_freq_factor: float, high_freq_factor: float,
                          original_max_position: int) -> torch.Tensor:
    """Not in the reference (its LlamaConfig has no rope_scaling,
    models/llama.py:9-20).  The rule of the "llama3" rope_scaling type, by
    wavelength lambda = 2 pi / inv_freq against the original context L:
      lambda < L / high_freq_factor            -> unchanged
      lambda > L / low_freq_factor             -> inv_freq / factor
      otherwise, s = (L / lambda - low) / (high - low)
                                               -> (1 - s) * inv_freq / factor + s * inv_freq
    """
    out = []
    for f in inv_freq.tolist():
        wavelen = 2.0 * math.pi / f
        if wavelen < original_max_position / high_freq_factor:
            out.append(f)
        elif wavelen > original_max_position / low_freq_factor:
            out.append(f / factor)
        else:
            s = (original_max_position / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
            out.append((1.0 - s) * f / factor + s * f)
    return torch.tensor(out, dtype=torch.float32)


def rope_cos_sin(positions: torch.Tensor, inv_freq: torch.Tensor):
    """python/lyapunov_engine/models/llama.py:186-194: freqs = outer(t, inv_freq);
    emb = cat((freqs, freqs), -1); cos = emb.cos(), sin = emb.sin() -- in 32-bit,
    but for the token's own position instead of arange(seq_len) (the reference
    restarts at 0 in every call, :206-207, which is wrong for a decoded token)."""
    freqs = torch.outer(positions.float(), inv_freq.float())
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """python/lyapunov_engine/models/llama.py:23-31: x1, x2 = halves of the last
    dimension; rotated = cat((-x2, x1)); out = x * cos + rotated * sin.
    x: [..., seq, head_dim]; cos, sin: [seq, head_dim]."""
    d = x.shape[-1]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    rotated = torch.cat((-x2, x1), dim=-1)
    return x * cos.to(x.dtype) + rotated * sin.to(x.dtype)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_positions: torch.Tensor,
              k_positions: torch.Tensor, scale: float | None = None, window: int = 0) -> torch.Tensor:
    """python/lyapunov_engine/ops.py:100-121: scale = 1/sqrt(head_dim); key/value
    heads repeated (repeat_interleave) so that query head h uses key/value head
    h // ratio; scores = q @ k^T * scale; causal mask; softmax; @ v.
    q [nh, Sq, hd]; k, v [nkv, Sk, hd].  The reference masks key index j > query
    index i with both counted from 0 (:113-118); here the mask compares absolute
    positions, so queries may start in the middle of a sequence.  ``window``
    (not in the reference): a query also does not see keys at or below
    position - window."""
    nh, nkv, hd = q.shape[0], k.shape[0], q.shape[-1]
    scale = 1.0 / math.sqrt(hd) if scale is None else scale
    if nh != nkv:
        k = k.repeat_interleave(nh // nkv, dim=0)
        v = v.repeat_interleave(nh // nkv, dim=0)
    scores = torch.matmul(q, k.transpose(-1, -2)) * scale
    qp, kp = q_positions.view(-1, 1), k_positions.view(1, -1)
    hidden = kp > qp
    if window > 0:
        hidden = hidden | (kp <= qp - window)
    scores = scores.masked_fill(hidden.unsqueeze(0), float("-inf"))
    return torch.matmul(torch.softmax(scores, dim=-1), v)


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """python/lyapunov_engine/ops.py:72-73: gate, up = chunk(2, -1); silu(gate) * up."""
    gate, up = gate_up.chunk(2, dim=-1)
    return torch.nn.functional.silu(gate) * up


def mlp(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """python/lyapunov_engine/models/llama.py:109-122 with the fused matrix of
    models/weight_loader.py:155-163 (cat([gate, up], dim=0)): down(swiglu(x @ Wgu^T))."""
    gate_up = x @ torch.cat([w_gate, w_up], dim=0).T
    return swiglu(gate_up) @ w_down.T


def attention_layer(x: torch.Tensor, positions: torch.Tensor, w: dict, prefix: str, cfg: dict,
                    inv_freq: torch.Tensor, window: int = 0) -> torch.Tensor:
    """python/lyapunov_engine/models/llama.py:50-106: q/k/v projections without
    bias, view [S, n, hd] -> [n, S, hd], rotation of q and k, causal attention,
    back to [S, nh * hd], o_proj."""
    S = x.shape[0]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = (x @ w[prefix + "q_proj.weight"].T).view(S, nh, hd).transpose(0, 1)
    k = (x @ w[prefix + "k_proj.weight"].T).view(S, nkv, hd).transpose(0, 1)
    v = (x @ w[prefix + "v_proj.weight"].T).view(S, nkv, hd).transpose(0, 1)
    cos, sin = rope_cos_sin(positions, inv_freq)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    out = attention(q, k, v, positions, positions, window=window)
    return out.transpose(0, 1).reshape(S, nh * hd) @ w[prefix + "o_proj.weight"].T


def decoder_layer(h: torch.Tensor, positions: torch.Tensor, w: dict, i: int, cfg: dict,
                  inv_freq: torch.Tensor) -> torch.Tensor:
    """python/lyapunov_engine/models/llama.py:147-165: h += attn(norm(h)); h += mlp(norm(h))."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    x = rms_norm(h, w[p + "input_layernorm.weight"], eps)
    h = h + attention_layer(x, positions, w, p + "self_attn.", cfg, inv_freq)
    x = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
    return h + mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])


def model_inv_freq(cfg: dict) -> torch.Tensor:
    inv_freq = rope_inv_freq(cfg["head_dim"], cfg["rope_theta"])
    rs = cfg.get("rope_scaling")
    if rs and rs.get("rope_type", rs.get("type")) == "llama3":
        inv_freq = llama3_scale_inv_freq(inv_freq, rs["factor"], rs["low_freq_factor"], rs["high_freq_factor"],
                                         rs["original_max_position_embeddings"])
    return inv_freq


def forward(w: dict, cfg: dict, tokens: list, dtype: torch.dtype = torch.float64) -> torch.Tensor:
    """python/lyapunov_engine/models/llama.py:196-225: embed, layers, final norm,
    lm_head, for one whole sequence at positions 0..S-1; logits for all
    positions, [S, vocab].  A tied head uses the embedding matrix (the
    reference's loader copies it into lm_head when the file has none,
    models/weight_loader.py:102-109)."""
    w = {k: v.to(dtype) for k, v in w.items()}
    ids = torch.tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    inv_freq = model_inv_freq(cfg)
    h = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        h = decoder_layer(h, positions, w, i, cfg, inv_freq)
    h = rms_norm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return h @ head.T


# -------------------------------------------------------------------- sampling
def sample_filter(logits: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """python/lyapunov_engine/engine/sampling.py:40-68: logits / T; top-k keeps
    values not below the k-th largest; top-p sorts descending, removes where the
    cumulative probability exceeds p, shifted right by one so that the token
    that crosses p stays and the first always stays; returns the probabilities
    the draw is made from."""
    b = logits.clone().double() / temperature
    if 0 < top_k < b.shape[-1]:
        kth = torch.topk(b, top_k).values[-1]
        b = torch.where(b < kth, torch.tensor(float("-inf"), dtype=b.dtype), b)
    if top_p < 1.0:
        sorted_logits, sorted_idx = torch.sort(b, descending=True)
        cum = torch.cumsum(torch.softmax(sorted_logits, dim=-1), dim=-1)
        remove = cum > top_p
        remove[1:] = remove[:-1].clone()
        remove[0] = False
        b[sorted_idx[remove]] = float("-inf")
    return torch.softmax(b, dim=-1)


def greedy(logits: torch.Tensor) -> int:
    """python/lyapunov_engine/engine/sampling.py:34-38: argmax when temperature < 1e-4."""
    return int(torch.argmax(logits).item())


def inverse_cdf(probs: torch.Tensor, u: float) -> int:
    """The engine's draw: the first token, in token order, at which the
    cumulative probability exceeds u (the reference draws with
    torch.multinomial, sampling.py:69, unseeded; the distribution is the same)."""
    cdf = torch.cumsum(probs.double(), dim=-1)
    idx = int(torch.searchsorted(cdf, torch.tensor(u * float(cdf[-1]), dtype=torch.float64), right=True).item())
    return min(idx, probs.numel() - 1)


# ----------------------------------------------------------------- model files
def read_model(folder: str):
    """-> (tensor dict in 32-bit, config dict), through the safetensors library."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as f:
        cfg = json.load(f)
    if "head_dim" not in cfg or cfg["head_dim"] is None:
        cfg["head_dim"] = cfg["hidden_size"] // cfg["num_attention_heads"]
    cfg.setdefault("num_key_value_heads", cfg["num_attention_heads"])
    w = {}
    for name in sorted(os.listdir(folder)):
        if name.endswith(".safetensors"):
            w.update(load_file(os.path.join(folder, name)))
    return {k: v.float() for k, v in w.items()}, cfg
