"""A plain, slow implementation of the Llama decoder for the tests.

Whole sequences, no cache, one function for each part, written from the
formulas of the reference (each function cites file:line under the reference
tree) and sharing no code with the engine: it reads config.json with ``json``
and the weights with the ``safetensors`` package.  Arithmetic is float64 by
default, so that what the engine's float32 path is compared with has no
rounding of its own worth mentioning.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# --- parts --------------------------------------------------------------------

def embedding(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """x[t, :] = table[ids[t], :]; no scaling, no position added.
    engine/kernels/embedding_lookup.cu:22-30; tools/references/reference_forward.py:363."""
    return table[ids]


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2) + eps) * w; eps joins the *mean* square.
    engine/kernels/rmsnorm.cu:26-40; tools/references/reference_forward.py:84-86."""
    mean_square = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * (1.0 / torch.sqrt(mean_square + eps)) * weight


def rope_angles(rotary_dim: int, positions: torch.Tensor, theta: float, dtype) -> torch.Tensor:
    """angle[t, p] = position[t] * theta^(-2p/dim) for p in [0, dim/2).
    engine/kernels/rope.cu:44-45; tools/references/reference_forward.py:89-93."""
    half = rotary_dim // 2
    inv_freq = 1.0 / (theta ** (torch.arange(half, dtype=dtype) * 2.0 / rotary_dim))
    return positions.to(dtype).unsqueeze(-1) * inv_freq


def rope(x: torch.Tensor, positions: torch.Tensor, theta: float, rotary_dim: Optional[int] = None) -> torch.Tensor:
    """x: [T, heads, d].  Rotate-half pairing: element p with element p + dim/2:
    lo' = lo cos - hi sin, hi' = hi cos + lo sin.
    engine/kernels/rope.cu:49-53; tools/references/reference_forward.py:96-104."""
    d = x.shape[-1]
    rd = d if rotary_dim is None else rotary_dim
    half = rd // 2
    ang = rope_angles(rd, positions, theta, x.dtype)
    cos, sin = torch.cos(ang).unsqueeze(1), torch.sin(ang).unsqueeze(1)   # [T, 1, half]
    lo, hi, rest = x[..., :half], x[..., half:rd], x[..., rd:]
    return torch.cat([lo * cos - hi * sin, hi * cos + lo * sin, rest], dim=-1)


def attention_scores(q: torch.Tensor, k: torch.Tensor, window: int = 0) -> torch.Tensor:
    """scores[h, i, j] = (q[i, h] . k[j, h // G]) / sqrt(d) for j <= i (and j > i - window
    if window > 0), -inf elsewhere.  The scale is applied after the dot product; query head
    h reads key/value head h // G with G = heads / kv_heads.
    engine/kernels/attention_qk.cu:25,34-35,49-54,63-68; tools/references/reference_forward.py:107-120."""
    t, n_heads, d = q.shape
    group = n_heads // k.shape[1]
    scores = torch.empty((n_heads, t, t), dtype=q.dtype)
    for h in range(n_heads):
        scores[h] = (q[:, h, :] @ k[:, h // group, :].T) * (1.0 / math.sqrt(d))
    i = torch.arange(t).unsqueeze(1)
    j = torch.arange(t).unsqueeze(0)
    hidden = j > i
    if window > 0:
        hidden = hidden | (j <= i - window)
    return scores.masked_fill(hidden.unsqueeze(0), float("-inf"))


def softmax_rows(scores: torch.Tensor) -> torch.Tensor:
    """p_j = exp(s_j - max) / sum; masked entries give exactly 0.
    engine/kernels/softmax.cu:28-42; tools/references/reference_forward.py:121."""
    m = scores.max(dim=-1, keepdim=True).values
    e = torch.exp(scores - m)
    return e / e.sum(dim=-1, keepdim=True)


def attention_output(probs: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """out[i, h, :] = sum_j probs[h, i, j] v[j, h // G, :].
    engine/kernels/attention_av.cu:32-45; tools/references/reference_forward.py:122."""
    n_heads, t, _ = probs.shape
    group = n_heads // v.shape[1]
    out = torch.empty((t, n_heads, v.shape[-1]), dtype=v.dtype)
    for h in range(n_heads):
        out[:, h, :] = probs[h] @ v[:, h // group, :]
    return out


def attention(q, k, v, window: int = 0) -> torch.Tensor:
    """tools/references/reference_forward.py:107-123."""
    return attention_output(softmax_rows(attention_scores(q, k, window)), v)


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """(g / (1 + exp(-g))) * u.  engine/kernels/swiglu.cu:22-23;
    tools/references/reference_forward.py:126-127."""
    return (gate / (1.0 + torch.exp(-gate))) * up


def argmax_lowest(row: torch.Tensor) -> int:
    """Index of the maximum; the lowest index on ties.
    engine/kernels/logits_argmax.cu:48-64."""
    m = row.max()
    return int(torch.nonzero(row == m)[0])


# --- the model ------------------------------------------------------------------

class PlainLlama:
    """Reads a model folder and computes logits for whole sequences.
    engine/src/model.cpp:522-615; tools/references/reference_forward.py:358-380."""

    def __init__(self, model_dir: str, dtype=torch.float64, round_weights_to_bf16: bool = False):
        from safetensors import safe_open
        with open(os.path.join(model_dir, "config.json")) as fh:
            c = json.load(fh)
        # tools/convert/convert_weights.py:35-46 (keys and defaults)
        self.vocab = c["vocab_size"]
        self.hidden = c["hidden_size"]
        self.layers = c["num_hidden_layers"]
        self.heads = c["num_attention_heads"]
        self.kv_heads = c.get("num_key_value_heads", self.heads)
        self.head_dim = c.get("head_dim") or self.hidden // self.heads
        self.inter = c["intermediate_size"]
        self.theta = float(c.get("rope_theta", 10000.0))
        self.eps = float(c.get("rms_norm_eps", 1e-5))
        self.tied = bool(c.get("tie_word_embeddings", False))
        self.dtype = dtype
        self.w: Dict[str, torch.Tensor] = {}
        with safe_open(os.path.join(model_dir, "model.safetensors"), "pt") as f:
            for name in f.keys():
                t = f.get_tensor(name)
                if round_weights_to_bf16:
                    t = t.to(torch.bfloat16)
                self.w[name] = t.to(dtype)
        if "lm_head.weight" not in self.w:
            assert self.tied, "no lm_head.weight and embeddings are not tied"
            self.w["lm_head.weight"] = self.w["model.embed_tokens.weight"]

    def hidden_states(self, ids: Sequence[int], position_offset: int = 0) -> torch.Tensor:
        w = self.w
        ids_t = torch.tensor(list(ids), dtype=torch.long)
        t = len(ids)
        positions = torch.arange(t) + position_offset
        x = embedding(w["model.embed_tokens.weight"], ids_t)
        for i in range(self.layers):
            p = f"model.layers.{i}."
            h = rmsnorm(x, w[p + "input_layernorm.weight"], self.eps)
            q = (h @ w[p + "self_attn.q_proj.weight"].T).view(t, self.heads, self.head_dim)
            k = (h @ w[p + "self_attn.k_proj.weight"].T).view(t, self.kv_heads, self.head_dim)
            v = (h @ w[p + "self_attn.v_proj.weight"].T).view(t, self.kv_heads, self.head_dim)
            q = rope(q, positions, self.theta)
            k = rope(k, positions, self.theta)
            o = attention(q, k, v).reshape(t, self.heads * self.head_dim)
            x = x + o @ w[p + "self_attn.o_proj.weight"].T
            h = rmsnorm(x, w[p + "post_attention_layernorm.weight"], self.eps)
            a = swiglu(h @ w[p + "mlp.gate_proj.weight"].T, h @ w[p + "mlp.up_proj.weight"].T)
            x = x + a @ w[p + "mlp.down_proj.weight"].T
        return x

    def logits(self, ids: Sequence[int], position_offset: int = 0) -> torch.Tensor:
        """[T, vocab] logits at every position of the sequence."""
        x = self.hidden_states(ids, position_offset)
        return rmsnorm(x, self.w["model.norm.weight"], self.eps) @ self.w["lm_head.weight"].T

    def greedy(self, prompt: Sequence[int], steps: int) -> List[int]:
        """Argmax decoding that recomputes the whole sequence every step.
        tools/references/reference_forward.py:382-391."""
        ids = list(prompt)
        out = []
        for _ in range(steps):
            nxt = argmax_lowest(self.logits(ids)[-1])
            out.append(nxt)
            ids.append(nxt)
        return out


# --- sampling -------------------------------------------------------------------

def sample_probabilities(logits: Sequence[float], temperature: float, top_k: int = 0,
                         top_p: float = 1.0) -> List[float]:
    """The distribution engine/src/sampler.cpp:36-103 draws from: softmax(l / T) restricted to
    the top_k likeliest (0 = all; lower id first on ties) and then to the fewest of those whose
    share of the kept mass reaches top_p, renormalized.  T <= 0 or top_k == 1 is the argmax."""
    n = len(logits)
    if temperature <= 0 or top_k == 1:
        best = max(range(n), key=lambda i: (logits[i], -i))
        return [1.0 if i == best else 0.0 for i in range(n)]
    m = max(logits)
    w = [math.exp((l - m) / temperature) for l in logits]
    order = sorted(range(n), key=lambda i: (-w[i], i))
    k = min(top_k, n) if top_k > 0 else n
    kept = order[:k]
    if top_p < 1.0:
        total = sum(w[i] for i in kept)
        cum, cut = 0.0, len(kept)
        for pos, i in enumerate(kept):
            cum += w[i]
            if cum >= top_p * total:
                cut = pos + 1
                break
        kept = kept[:cut]
    total = sum(w[i] for i in kept)
    keep = set(kept)
    return [w[i] / total if i in keep else 0.0 for i in range(n)]
