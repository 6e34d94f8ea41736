"""A plain, slow implementation of the Qwen2.5-VL text decoder, written from the reference's
formulas: whole sequences, no cache, float32 on the CPU, one function for each part.  It shares
no code with the engine (it reads config.json and the safetensors file on its own) and is what
the engine's logits are compared with.  Each function cites the reference lines it follows.
"""

from __future__ import annotations

import json
import os
from typing import Dict, List, Optional, Sequence

import torch


# --------------------------------------------------------------------------------------------
# configuration and weights, read independently of the engine
# --------------------------------------------------------------------------------------------
def plain_read_config(model_dir: str) -> dict:
    """The decoder's fields as a flat dict (reference config.py:163-201: text_config holds the
    sizes; rope constants may sit in rope_scaling / rope_parameters; tie flag from the top)."""
    with open(os.path.join(model_dir, "config.json")) as fh:
        raw = json.load(fh)
    text = dict(raw.get("text_config") or raw)
    for key in ("rope_scaling", "rope_parameters"):
        for holder in (raw, raw.get("text_config") or {}):
            block = holder.get(key)
            if isinstance(block, dict):
                for name in ("mrope_section", "rope_theta"):
                    if name in block and name not in text:
                        text[name] = block[name]
    for name in ("rope_theta", "mrope_section", "tie_word_embeddings", "sliding_window", "use_sliding_window",
                 "max_window_layers", "layer_types"):
        if name in raw and name not in text:
            text[name] = raw[name]
    text.setdefault("tie_word_embeddings", True)
    text.setdefault("rms_norm_eps", 1e-6)        # reference config.py:88
    text.setdefault("rope_theta", 1_000_000.0)   # reference config.py:89
    text.setdefault("num_key_value_heads", text["num_attention_heads"])
    text.setdefault("head_dim", text["hidden_size"] // text["num_attention_heads"])  # reference config.py:97-99
    return text


def plain_layer_windows(cfg: dict) -> List[Optional[int]]:
    """Window of each layer.  Layers with index >= max_window_layers are windowed when
    use_sliding_window is set; an explicit layer_types list wins."""
    n = cfg["num_hidden_layers"]
    if cfg.get("layer_types"):
        return [cfg["sliding_window"] if t == "sliding_attention" else None for t in cfg["layer_types"]]
    if not cfg.get("use_sliding_window"):
        return [None] * n
    first = cfg.get("max_window_layers")
    first = n if first is None else first
    return [cfg["sliding_window"] if i >= first else None for i in range(n)]


def plain_read_weights(model_dir: str) -> Dict[str, torch.Tensor]:
    """Tensors by canonical name (``layers.0...``), float32.  Both checkpoint layouts are taken
    and the vision tower is skipped (reference model.py:52-73)."""
    from safetensors import safe_open

    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            rest = name[len("model."):] if name.startswith("model.") else name
            if rest.startswith("visual."):
                continue
            if rest.startswith("language_model."):
                rest = rest[len("language_model."):]
            out[rest] = f.get_tensor(name).to(torch.float32)
    return out


# --------------------------------------------------------------------------------------------
# the parts
# --------------------------------------------------------------------------------------------
def _keep(x: torch.Tensor) -> torch.Tensor:
    return x


def as_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 and back: what storing a float32 value in bfloat16 does to it."""
    return x.to(torch.bfloat16).to(torch.float32)


def plain_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """reference layers.py:27-31: x * rsqrt(mean(x^2) + eps), then times the weight."""
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return xf * weight


def plain_inv_freq(dim: int, theta: float) -> torch.Tensor:
    """reference rope.py:32-33."""
    idx = torch.arange(0, dim, 2, dtype=torch.float32)
    return 1.0 / (theta ** (idx / dim))


def plain_rotate_half(x: torch.Tensor) -> torch.Tensor:
    """reference rope.py:36-40: (-second half, first half)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def plain_mrope_cos_sin(position_ids: torch.Tensor, inv_freq: torch.Tensor):
    """reference rope.py:48-68.  position_ids [3, T] -> cos, sin of [3, T, head_dim]."""
    freqs = position_ids.to(torch.float32)[:, :, None] * inv_freq.to(torch.float32)[None, None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def plain_apply_mrope(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                      mrope_section: Sequence[int]):
    """reference rope.py:71-96.  q [heads, T, hd], k [kv_heads, T, hd]; cos/sin [3, T, hd].
    The section list is repeated (not each entry doubled); chunk i reads row i % 3."""
    sections = [int(s) for s in mrope_section] * 2
    if sum(sections) != cos.shape[-1]:
        raise ValueError("mrope_section does not cover the head size")
    cos_sel = torch.cat([m[i % 3] for i, m in enumerate(cos.split(sections, dim=-1))], dim=-1)
    sin_sel = torch.cat([m[i % 3] for i, m in enumerate(sin.split(sections, dim=-1))], dim=-1)
    return q * cos_sel + plain_rotate_half(q) * sin_sel, k * cos_sel + plain_rotate_half(k) * sin_sel


def plain_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                    window: Optional[int] = None) -> torch.Tensor:
    """reference attention.py:425-436 (explicit softmax) with the causal mask of
    attention.py:366-372: key j is visible to query i iff j <= i, and with a window iff also
    i - j < window.  GQA: query head h reads key head h // (heads / kv_heads)
    (reference attention.py:143-148).  q [heads, T, hd]; k, v [kv_heads, T, hd]."""
    heads, t, _ = q.shape
    groups = heads // k.shape[0]
    kk = k.repeat_interleave(groups, dim=0).float()
    vv = v.repeat_interleave(groups, dim=0).float()
    out = []
    rows = 1024   # queries are taken a slice at a time, only so that the score matrix of a long sequence fits memory
    for lo in range(0, t, rows):
        hi = min(t, lo + rows)
        scores = torch.matmul(q[:, lo:hi].float(), kk[:, :hi].transpose(-2, -1)) * scale
        i = torch.arange(lo, hi)[:, None]
        j = torch.arange(hi)[None, :]
        allowed = j <= i
        if window is not None:
            allowed = allowed & (i - j < window)
        scores = scores.masked_fill(~allowed, float("-inf"))
        out.append(torch.matmul(torch.softmax(scores, dim=-1), vv[:, :hi]))
    return torch.cat(out, dim=1)


def plain_mlp(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, store=_keep) -> torch.Tensor:
    """reference text.py:65-66: down(silu(gate(x)) * up(x)), no biases."""
    lin = torch.nn.functional.linear
    return lin(store(torch.nn.functional.silu(store(lin(x, gate))) * store(lin(x, up))), down)


def plain_attention_layer(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, cfg: dict,
                          position_ids: torch.Tensor, window: Optional[int], store=_keep) -> torch.Tensor:
    """reference text.py:85-90 (projections, heads), :118 (rotation), :78 (scale), :177-178.
    ``store`` is applied where a bfloat16 run stores a value: rotated queries and keys, values,
    the attention output (reference text.py:125-126 writes k and v to the cache in its dtype)."""
    t = x.shape[0]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    lin = torch.nn.functional.linear
    q = lin(x, w[prefix + "q_proj.weight"], w[prefix + "q_proj.bias"]).view(t, nh, hd).transpose(0, 1)
    k = lin(x, w[prefix + "k_proj.weight"], w[prefix + "k_proj.bias"]).view(t, nkv, hd).transpose(0, 1)
    v = lin(x, w[prefix + "v_proj.weight"], w[prefix + "v_proj.bias"]).view(t, nkv, hd).transpose(0, 1)
    cos, sin = plain_mrope_cos_sin(position_ids, plain_inv_freq(hd, cfg["rope_theta"]))
    q, k = plain_apply_mrope(q, k, cos, sin, cfg["mrope_section"])
    o = store(plain_attention(store(q), store(k), store(v), hd ** -0.5, window))
    return lin(o.transpose(0, 1).reshape(t, nh * hd), w[prefix + "o_proj.weight"])


def plain_forward(cfg: dict, w: Dict[str, torch.Tensor], token_ids: Sequence[int],
                  position_ids: Optional[torch.Tensor] = None, store=_keep) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence (reference text.py:196-206, 264-279; model.py:84-86,
    200-202).  Text positions: 0..T-1 on all three rows (reference rope.py:194-197).

    ``store`` models a run whose activations are stored in a narrower type: it is applied to the
    normalised activations, to q, k, v and the attention output, and to the feed-forward's
    inner values, i.e. to every operand of a matrix product and to what the cache holds (the
    reference runs all of these in its model dtype).  The residual sum, the norms' statistics
    and the logits stay float32.  ``as_bfloat16`` gives what a bfloat16 run can be held to."""
    ids = torch.tensor(list(token_ids), dtype=torch.long)
    t = ids.shape[0]
    if position_ids is None:
        position_ids = torch.arange(t)[None, :].expand(3, t)
    position_ids = torch.as_tensor(position_ids, dtype=torch.long)
    windows = plain_layer_windows(cfg)
    eps = cfg["rms_norm_eps"]
    h = w["embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        p = f"layers.{i}."
        a = plain_attention_layer(store(plain_rmsnorm(h, w[p + "input_layernorm.weight"], eps)), w,
                                  p + "self_attn.", cfg, position_ids, windows[i], store)
        h = h + a
        m = plain_mlp(store(plain_rmsnorm(h, w[p + "post_attention_layernorm.weight"], eps)),
                      w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"],
                      store)
        h = h + m
    h = store(plain_rmsnorm(h, w["norm.weight"], eps))
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["embed_tokens.weight"]
    return torch.nn.functional.linear(h, head)


def plain_model_logits(model_dir: str, token_ids: Sequence[int], position_ids=None, store=_keep) -> torch.Tensor:
    return plain_forward(plain_read_config(model_dir), plain_read_weights(model_dir), token_ids, position_ids, store)


# --------------------------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------------------------
def plain_penalties(logits: torch.Tensor, prev_ids: Sequence[int], repetition: float = 1.0, presence: float = 0.0,
                    frequency: float = 0.0) -> torch.Tensor:
    """reference sampling.py:44-64: over the output tokens so far; seen logits > 0 are divided by
    the repetition penalty, the others multiplied; then presence and frequency are subtracted."""
    out = logits.clone().float()
    if not prev_ids:
        return out
    counts = torch.bincount(torch.tensor(list(prev_ids)), minlength=out.shape[-1]).float()
    seen = counts > 0
    if repetition != 1.0:
        out[seen] = torch.where(out[seen] > 0, out[seen] / repetition, out[seen] * repetition)
    out = out - presence * seen.float() - frequency * counts
    return out


def plain_filtered_probs(logits: torch.Tensor, temperature: float, top_k: int = -1, top_p: float = 1.0,
                         min_p: float = 0.0) -> torch.Tensor:
    """reference sampling.py:72-103: scores / T; top-k keeps scores >= the k-th largest; min-p drops
    probabilities below min_p * max; top-p keeps the smallest sorted prefix whose mass reaches top_p
    (the crossing token is kept); softmax of what is left."""
    scores = logits.float() / temperature
    if top_k and top_k > 0:
        kth = torch.topk(scores, min(top_k, scores.numel())).values[-1]
        scores = torch.where(scores < kth, torch.full_like(scores, float("-inf")), scores)
    if min_p > 0:
        probs = torch.softmax(scores, dim=-1)
        scores = torch.where(probs < min_p * probs.max(), torch.full_like(scores, float("-inf")), scores)
    if top_p < 1.0:
        sorted_scores, order = torch.sort(scores, descending=True)
        cumulative = torch.cumsum(torch.softmax(sorted_scores, dim=-1), dim=-1)
        crossing = (cumulative >= top_p).nonzero(as_tuple=True)[0]
        keep = torch.zeros_like(cumulative, dtype=torch.bool)
        keep[0] = True
        if crossing.numel():
            keep[: int(crossing[0]) + 1] = True
        else:
            keep[:] = True
        filtered = torch.full_like(sorted_scores, float("-inf"))
        filtered[keep] = sorted_scores[keep]
        scores = torch.empty_like(scores).scatter_(0, order, filtered)
    return torch.softmax(scores, dim=-1)
