"""A plain, slow Qwen3 dense decoder: whole sequences, no cache, one function per
part, float64 on the CPU.  It shares no code with ``pulse_infer_amd``; it reads a
model folder with ``json`` and the ``safetensors`` package, and is written from
the reference's formulas (file:line in each docstring; paths are relative to the
reference's root).  Tests compare the engine with it.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

DT = torch.float64


def embedding(table: torch.Tensor, ids: List[int]) -> torch.Tensor:
    """h[t, :] = table[ids[t], :]  (src/layer/embedding.cpp:132-153,
    include/pulse/ops/kernels/embedding_kernel.hpp:16-25)."""
    return table[torch.tensor(ids, dtype=torch.long)]


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * (1 / sqrt(mean(x^2) + eps)) * w over the last axis; the weight multiplies after
    the normalisation  (include/pulse/ops/kernels/rmsnorm_kernel.hpp:17-35,
    src/ops/kernels/cuda/rmsnorm_kernel.cu:97-157)."""
    inv = 1.0 / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return x * inv * weight


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y = x W^T, W stored [out, in], no bias  (src/layer/linear.cpp:213,
    src/ops/kernels/cuda/matmul_kernel.cu:63-67)."""
    return x @ weight.transpose(0, 1)


def rope(x: torch.Tensor, positions: List[int], theta: float, rotary_dim: Optional[int] = None,
         pairing: str = "interleaved") -> torch.Tensor:
    """Rotate pairs of channels of x [T, heads, d] by angle = position / theta^(2i / rotary_dim).

    The reference pairs ADJACENT channels (2i, 2i+1):
      out[2i]   = x[2i] cos - x[2i+1] sin
      out[2i+1] = x[2i] sin + x[2i+1] cos
    (src/ops/rope.cpp:55-69, src/ops/kernels/cuda/rope_kernel.cu:100-126); channels at or beyond
    rotary_dim are copied (rope_kernel.cu:95-98).  ``pairing="half"`` pairs (i, i + rotary_dim/2).
    """
    t, heads, d = x.shape
    rot = d if rotary_dim is None else rotary_dim
    out = x.clone()
    pos = torch.tensor(positions, dtype=DT).view(t, 1)
    for i in range(rot // 2):
        angle = pos / (theta ** ((2.0 * i) / rot))
        c, s = torch.cos(angle), torch.sin(angle)
        a, b = (2 * i, 2 * i + 1) if pairing == "interleaved" else (i, i + rot // 2)
        xa, xb = x[:, :, a], x[:, :, b]
        out[:, :, a] = xa * c - xb * s
        out[:, :, b] = xa * s + xb * c
    return out


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     window: Optional[int] = None, q_positions: Optional[List[int]] = None) -> torch.Tensor:
    """Per query t and head h: scores over keys j <= position(t) (and j > position(t) - window when a
    window is set), s_j = (q . k_j) * scale, softmax with the maximum subtracted, o = sum p_j v_j.
    Query head h reads kv head h // (nq // nkv)
    (src/ops/kernels/cuda/paged_attention.cu:61-70 head mapping, :88-137 scores/softmax/sum;
    include/pulse/ops/kernels/mha_kernel.hpp:47-87 for the dense twin).
    q [T, nq, d]; k, v [S, nkv, d] hold keys of positions 0..S-1; q_positions default 0..T-1 (T == S)."""
    tq, nq, d = q.shape
    s_len, nkv, _ = k.shape
    group = nq // nkv
    if q_positions is None:
        q_positions = list(range(tq))
    out = torch.zeros_like(q)
    for t in range(tq):
        p = q_positions[t]
        lo = 0 if window is None else max(0, p - window + 1)
        for h in range(nq):
            g = h // group
            keys = k[lo:p + 1, g, :]
            vals = v[lo:p + 1, g, :]
            scores = (keys @ q[t, h, :]) * scale
            scores = scores - scores.max()
            w = torch.exp(scores)
            w = w / w.sum()
            out[t, h, :] = w @ vals
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x))  (src/ops/kernels/cuda/silu_kernel.cu:20-30, include/pulse/ops/kernels/silu_kernel.hpp)."""
    return x / (1.0 + torch.exp(-x))


def gated_mlp(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """down( silu(gate(x)) * up(x) )  (src/model/qwen3/model.cpp:893-913)."""
    return linear(silu(linear(x, w_gate)) * linear(x, w_up), w_down)


class PlainQwen3:
    """The whole decoder on whole sequences (src/model/qwen3/model.cpp:750-926 per layer, :1283-1371 around)."""

    def __init__(self, config: Dict, weights: Dict[str, torch.Tensor], pairing: str = "interleaved",
                 windows: Optional[List[Optional[int]]] = None):
        """``windows``: an attention window per layer (None: all keys).  The reference has no windows; they are a
        parameter of ``causal_attention`` here and an option of the engine there."""
        self.c = config
        self.w = {k: v.to(DT) for k, v in weights.items()}
        self.pairing = pairing
        self.windows = windows

    @classmethod
    def from_folder(cls, folder: str, pairing: str = "interleaved",
                    windows: Optional[List[Optional[int]]] = None) -> "PlainQwen3":
        from safetensors.torch import load_file

        with open(os.path.join(folder, "config.json")) as fh:
            config = json.load(fh)
        weights: Dict[str, torch.Tensor] = {}
        for name in sorted(os.listdir(folder)):
            if name.endswith(".safetensors"):
                weights.update(load_file(os.path.join(folder, name)))
        return cls(config, weights, pairing, windows)

    def layer_window(self, layer: int) -> Optional[int]:
        return self.windows[layer] if self.windows is not None else None

    def layer(self, h: torch.Tensor, index: int, positions: List[int],
              rows: Optional[List[int]] = None) -> torch.Tensor:
        """One layer on the whole sequence.  ``rows``: the layer's output is wanted for these places only; keys and
        values are still those of every position, queries and everything after them only of the rows."""
        c, w = self.c, self.w
        p = f"model.layers.{index}."
        nq, nkv = c["num_attention_heads"], c["num_key_value_heads"]
        d = c.get("head_dim", c["hidden_size"] // nq)
        eps = c["rms_norm_eps"]
        t = h.shape[0]
        sel = list(range(t)) if rows is None else list(rows)
        sel_pos = [positions[i] for i in sel]
        # pre-norm stands before the projections (model.cpp:779)
        a = rms_norm(h, w[p + "input_layernorm.weight"], eps)
        q = linear(a[sel], w[p + "self_attn.q_proj.weight"]).view(len(sel), nq, d)     # model.cpp:784-813
        k = linear(a, w[p + "self_attn.k_proj.weight"]).view(t, nkv, d)
        v = linear(a, w[p + "self_attn.v_proj.weight"]).view(t, nkv, d)
        # per-head norm over d, after projection and before rotation; v untouched (model.cpp:815-838)
        q = rms_norm(q, w[p + "self_attn.q_norm.weight"], eps)
        k = rms_norm(k, w[p + "self_attn.k_norm.weight"], eps)
        q = rope(q, sel_pos, c["rope_theta"], d, self.pairing)
        k = rope(k, positions, c["rope_theta"], d, self.pairing)
        # keys are indexed by their place in the sequence; positions only enter through the rotation
        o = causal_attention(q, k, v, 1.0 / math.sqrt(d), self.layer_window(index), sel)  # scale: paged_attention.cu:108
        h = h[sel] + linear(o.reshape(len(sel), nq * d), w[p + "self_attn.o_proj.weight"])   # model.cpp:875-886
        m = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)                       # model.cpp:888
        h = h + gated_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                          w[p + "mlp.down_proj.weight"])                                    # model.cpp:893-923
        return h

    def hidden(self, ids: List[int], rows: Optional[List[int]] = None) -> torch.Tensor:
        positions = list(range(len(ids)))
        h = embedding(self.w["model.embed_tokens.weight"], ids)
        last = self.c["num_hidden_layers"] - 1
        for i in range(last + 1):
            h = self.layer(h, i, positions, rows if i == last else None)
        return h

    def logits(self, ids: List[int], rows: Optional[List[int]] = None) -> torch.Tensor:
        """[T, V] logits of every position, or [len(rows), V] of the places in ``rows`` (the last layer then computes
        queries for those only)  (model.cpp:1305-1371: final norm, then the head; lm_head.weight if present, else the
        embedding table when tied)."""
        h = rms_norm(self.hidden(ids, rows), self.w["model.norm.weight"], self.c["rms_norm_eps"])
        head = self.w.get("lm_head.weight")
        if head is None:
            if not self.c.get("tie_word_embeddings", False):
                raise KeyError("lm_head.weight is missing and embeddings are not tied")
            head = self.w["model.embed_tokens.weight"]
        return linear(h, head)

    def greedy(self, prompt: List[int], steps: int) -> List[int]:
        """Greedy continuation, recomputing the whole sequence each time; lowest index wins ties
        (src/scheduler/continuous_batch_engine.cpp:20-62)."""
        ids = list(prompt)
        out = []
        for _ in range(steps):
            row = self.logits(ids)[-1]
            tok = int(torch.argmax(row))  # torch returns the first maximal index
            out.append(tok)
            ids.append(tok)
        return out
