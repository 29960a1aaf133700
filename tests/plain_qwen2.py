"""Plain, slow Qwen2.5 forward pass used as the oracle of the test-suite.

Whole sequences, no cache, one function per part, CPU only.  It shares no code
with ``torchlet_amd``: it reads ``config.json`` and ``model.safetensors`` by
itself and is written from the formulas of the reference's first version
(``/root/reference/src/torchlet/v00_full_recompute``), cited function by function.

Every function takes and returns ``torch`` CPU tensors of one floating dtype
(``float64`` by default, so that the oracle's own rounding is far below the
engine's 32-bit rounding).

The attention window is not in the reference (it never reads the ``sliding_window``
keys); ``window=None`` is the reference's behaviour.  With a window ``W`` a query at
position ``t`` sees the keys ``t-W < s <= t``: parity unpinned, the definition is
this file's.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------- parts

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``x * rsqrt(mean(x^2) + eps) * weight``; eps inside the root, weight last.

    Reference: v00_full_recompute/layer/rms_norm.py:11-13.
    """
    mean_sq = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(mean_sq + eps) * weight


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``x @ weight.T + bias`` with ``weight`` stored ``[out, in]`` (``nn.Linear``).

    Reference: v00_full_recompute/layer/gqa.py:34-39 (q/k/v/o projections).
    """
    y = x @ weight.transpose(-1, -2)
    if bias is not None:
        y = y + bias
    return y


def rope_angles(positions: torch.Tensor, head_dim: int, theta: float) -> torch.Tensor:
    """Angles ``[len(positions), head_dim/2]``: ``pos * theta**(-2j/head_dim)``.

    The inverse frequencies and the product are taken in float32 on the host, as the reference's
    table is when its module is constructed (v00_full_recompute/layer/rope.py:29-35), then moved to
    where the positions are and widened by the caller.  (A power taken by another device's routine
    may differ in its last bit, which a position of several thousand turns into 1e-4 of an angle.)
    """
    j = torch.arange(0, head_dim, 2, dtype=torch.float32)
    inv_freq = 1.0 / (theta ** (j / head_dim))
    return torch.outer(positions.to(device="cpu", dtype=torch.float32), inv_freq).to(positions.device)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """``[-x2, x1]`` with ``x1``/``x2`` the first/second half of the last axis.

    Reference: v00_full_recompute/layer/rope.py:63-75.
    """
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def rope_apply(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Split-half rotation of ``x [heads, tokens, head_dim]`` at ``positions [tokens]``.

    ``x*cos + rotate_half(x)*sin`` with ``cos/sin = cat(angle, angle)``.
    Reference: v00_full_recompute/layer/rope.py:46-61.
    """
    angle = rope_angles(positions, x.shape[-1], theta)
    emb = torch.cat((angle, angle), dim=-1)
    cos = emb.cos().to(x.dtype)
    sin = emb.sin().to(x.dtype)
    return x * cos + rotate_half(x) * sin


def attention_weights(q: torch.Tensor, k: torch.Tensor, window: int | None = None) -> torch.Tensor:
    """Causal softmax weights ``[heads, T, T]`` of ``q, k [heads, T, head_dim]``.

    Order of the reference: scores, ``-inf`` above the diagonal, divide by
    ``sqrt(head_dim)``, softmax (v00_full_recompute/layer/gqa.py:69-83).
    """
    t = q.shape[-2]
    scores = q @ k.transpose(-1, -2)
    idx = torch.arange(t, device=q.device)
    hidden = idx[None, :] > idx[:, None]
    if window is not None:
        hidden = hidden | (idx[None, :] <= idx[:, None] - window)
    scores = scores.masked_fill(hidden, -torch.inf)
    return torch.softmax(scores / k.shape[-1] ** 0.5, dim=-1)


def gqa_attention(
    h: torch.Tensor,
    w: dict[str, torch.Tensor],
    *,
    num_heads: int,
    num_kv_heads: int,
    head_dim: int,
    theta: float,
    positions: torch.Tensor,
    window: int | None = None,
    stored=lambda t: t,
) -> torch.Tensor:
    """Grouped-query attention of one request, ``h [T, hidden] -> [T, hidden]``.

    q/k/v projections with optional bias, head split (feature = head*head_dim + d),
    rotation of q and k, K/V repeated ``num_heads/num_kv_heads`` times so that query
    head ``i`` reads KV head ``i // group``, causal softmax, output projection without
    bias.  Reference: v00_full_recompute/layer/gqa.py:43-91.

    ``stored`` is applied to every tensor that an implementation in separate steps would
    write to memory between them (projections, rotated heads, the mixed heads, the output);
    a test passes a rounding there to see how much such roundings alone can move the result.
    """
    t = h.shape[0]
    q = stored(linear(h, w["q_proj.weight"], w.get("q_proj.bias")))
    k = stored(linear(h, w["k_proj.weight"], w.get("k_proj.bias")))
    v = stored(linear(h, w["v_proj.weight"], w.get("v_proj.bias")))
    q = q.view(t, num_heads, head_dim).transpose(0, 1)
    k = k.view(t, num_kv_heads, head_dim).transpose(0, 1)
    v = v.view(t, num_kv_heads, head_dim).transpose(0, 1)
    q = stored(rope_apply(q, positions, theta))
    k = stored(rope_apply(k, positions, theta))
    group = num_heads // num_kv_heads
    k = k.repeat_interleave(group, dim=0)
    v = v.repeat_interleave(group, dim=0)
    weights = attention_weights(q, k, window)
    ctx = stored((weights @ v).transpose(0, 1).contiguous().view(t, num_heads * head_dim))
    return stored(linear(ctx, w["o_proj.weight"]))


def swiglu_ffn(h: torch.Tensor, w: dict[str, torch.Tensor], stored=lambda t: t) -> torch.Tensor:
    """``down(silu(gate(h)) * up(h))``, no biases.

    Reference: v00_full_recompute/layer/ffn_swiglu.py:8-14.  ``stored``: see :func:`gqa_attention`.
    """
    gate = linear(h, w["gate_proj.weight"])
    up = linear(h, w["up_proj.weight"])
    return stored(linear(stored(torch.nn.functional.silu(gate) * up), w["down_proj.weight"]))


def block(x: torch.Tensor, w: dict[str, torch.Tensor], cfg: "PlainConfig", layer: int, positions: torch.Tensor,
          stored=lambda t: t) -> torch.Tensor:
    """Pre-norm residual block: ``x += attn(norm1(x)); x += ffn(norm2(x))``.

    Reference: v00_full_recompute/layer/transformer_block.py:34-37.
    """
    attn_w = _sub(w, "self_attn.")
    x = x + gqa_attention(
        stored(rms_norm(x, w["input_layernorm.weight"], cfg.eps)),
        attn_w,
        num_heads=cfg.num_heads,
        num_kv_heads=cfg.num_kv_heads,
        head_dim=cfg.head_dim,
        theta=cfg.theta,
        positions=positions,
        window=cfg.window_of(layer),
        stored=stored,
    )
    x = x + swiglu_ffn(stored(rms_norm(x, w["post_attention_layernorm.weight"], cfg.eps)), _sub(w, "mlp."), stored)
    return x


# --------------------------------------------------------------------------- model

class PlainConfig:
    """The keys the reference reads, with its defaults.

    Reference: v00_full_recompute/model/qwen2_5.py:13-36,75.  ``head_dim`` (default
    ``hidden // heads``) and the three window keys are additions the reference does
    not read.
    """

    def __init__(self, d: dict):
        self.vocab = d["vocab_size"]
        self.hidden = d["hidden_size"]
        self.layers = d["num_hidden_layers"]
        self.num_heads = d["num_attention_heads"]
        self.num_kv_heads = d.get("num_key_value_heads", self.num_heads)
        self.intermediate = d["intermediate_size"]
        self.eps = d.get("rms_norm_eps", 1e-6)
        self.bias = d.get("attention_bias", True)
        rope_parameters = d.get("rope_parameters")
        if isinstance(rope_parameters, dict) and "rope_theta" in rope_parameters:
            self.theta = rope_parameters["rope_theta"]
        else:
            self.theta = d.get("rope_theta", 1_000_000.0)
        self.tied = d.get("tie_word_embeddings", False)
        self.head_dim = d.get("head_dim") or self.hidden // self.num_heads
        self.use_window = bool(d.get("use_sliding_window", False))
        self.window = d.get("sliding_window")
        self.max_window_layers = d.get("max_window_layers", self.layers)

    def window_of(self, layer: int) -> int | None:
        """Layers from ``max_window_layers`` on are windowed when the window is on."""
        if self.use_window and self.window is not None and layer >= self.max_window_layers:
            return int(self.window)
        return None


def _sub(w: dict[str, torch.Tensor], prefix: str) -> dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def load_folder(folder: str | Path, dtype: torch.dtype = torch.float64):
    """Read ``config.json`` and every ``*.safetensors`` of a folder (sorted, merged).

    Reference: v00_full_recompute/llm.py:25-46.
    """
    folder = Path(folder)
    cfg = PlainConfig(json.loads((folder / "config.json").read_text()))
    weights: dict[str, torch.Tensor] = {}
    for path in sorted(folder.glob("*.safetensors")):
        with safe_open(str(path), framework="pt") as f:
            for name in f.keys():
                weights[name] = f.get_tensor(name).to(dtype)
    return cfg, weights


def forward(cfg: PlainConfig, weights: dict[str, torch.Tensor], token_ids: list[int], first_position: int = 0,
            stored=lambda t: t, last: int | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole request (``last``: of its last that many positions only).

    embedding, ``layers`` blocks, final norm, LM head without bias (the embedding
    matrix itself when tied).  Reference: v00_full_recompute/model/qwen2_5.py:55-82.
    ``first_position`` shifts every position by a constant (used by an invariance test).
    """
    device = weights["model.embed_tokens.weight"].device
    ids = torch.tensor(token_ids, dtype=torch.long, device=device)
    positions = torch.arange(len(token_ids), device=device) + first_position
    x = weights["model.embed_tokens.weight"][ids]
    for i in range(cfg.layers):
        x = block(x, _sub(weights, f"model.layers.{i}."), cfg, i, positions, stored)
    if last is not None:
        x = x[-last:]
    x = stored(rms_norm(x, weights["model.norm.weight"], cfg.eps))
    head = weights["model.embed_tokens.weight"] if cfg.tied else weights["lm_head.weight"]
    return linear(x, head)


def greedy(cfg: PlainConfig, weights: dict[str, torch.Tensor], prompt: list[int], max_new_tokens: int, stop_ids=()) -> list[int]:
    """Recompute-everything greedy loop; a stop id ends it and is not kept.

    Reference: v00_full_recompute/llm.py:47-87.
    """
    ids = list(prompt)
    out: list[int] = []
    for _ in range(max_new_tokens):
        tok = int(forward(cfg, weights, ids)[-1].argmax())
        if tok in stop_ids:
            break
        out.append(tok)
        ids.append(tok)
    return out


def softmax_temperature(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """Probabilities ``softmax(logits / temperature)`` (this file's definition; the
    reference samples greedily only, v00_full_recompute/llm.py:89-90)."""
    return torch.softmax(logits.double() / temperature, dim=-1)
