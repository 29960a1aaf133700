"""CPU stand-ins for the HIP entry points, for tests only.

The product has no CPU path.  These functions have the signatures and the semantics of
``torchlet_amd.kernels.ops`` (same operands, same in-place outputs, same block-table and
tile conventions) so that the engine's host logic -- cache manager, step function,
scheduler, trace replay -- can be exercised on a machine without a GPU by patching them
over the real module (see the ``cpu_ops`` fixture).  GPU tests never use this file.
"""
import math

import torch

ATTENTION_ROWS = 16


def attention_tile_tokens(num_heads, num_kv_heads):
    group = num_heads // num_kv_heads
    return max(1, ATTENTION_ROWS // min(group, ATTENTION_ROWS))


def load(names):
    pass


def embedding(token_ids, table, out, scale=1.0):
    out.copy_(table.float()[token_ids.long()] * scale)


def add_rmsnorm(residual, pending, weight, eps, out, rows=None, gain=1.0):
    if pending is not None and pending.dim() == 3:
        pending = pending.sum(0)
    if rows is None:
        if pending is not None:
            residual += pending.float()
        r = residual
    else:
        idx = rows.long()
        r = residual[idx] + (pending[idx].float() if pending is not None else 0)
    y = r * (torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps) * gain) * weight.float()
    out.copy_(y.to(out.dtype))


def linear(x, weight, bias, out, general=False):
    y = x.float() @ weight.float().T
    if bias is not None:
        y = y + bias.float()
    out.copy_(y.to(out.dtype))


def linear_rope_cache_write(*args, **kwargs):
    return False          # not fused here: the caller runs the product and the rotation one after the other


def rope_cache_write(qkv, q_heads, kv_heads, head_dim, rot_heads, positions, inv_freq,
                     token_req=None, block_table=None, k_plane=None, v_plane=None, page_size=0, pairs=False, parts=None, bias=None):
    T = qkv.shape[0]
    if parts is not None:
        total = parts.sum(0) + (bias.float() if bias is not None else 0.0)
        qkv[:, : total.shape[1]] = total.to(qkv.dtype)
    x = qkv[:, : (q_heads + kv_heads) * head_dim].float().view(T, q_heads + kv_heads, head_dim)
    if inv_freq is not None:
        ang = positions.float()[:, None] * inv_freq[None, :]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        half = head_dim // 2
        if pairs:
            x1, x2 = x[:, :rot_heads, 0::2], x[:, :rot_heads, 1::2]
            turned = torch.stack((x1 * c - x2 * s, x2 * c + x1 * s), -1).reshape(T, rot_heads, head_dim)
        else:
            x1, x2 = x[:, :rot_heads, :half], x[:, :rot_heads, half:]
            turned = torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), -1)
        x = torch.cat((turned, x[:, rot_heads:]), 1)
        qkv[:, : (q_heads + kv_heads) * head_dim] = x.reshape(T, -1).to(qkv.dtype)
    if k_plane is not None:
        k = qkv[:, q_heads * head_dim: (q_heads + kv_heads) * head_dim].view(T, kv_heads, head_dim)
        v = qkv[:, (q_heads + kv_heads) * head_dim: (q_heads + 2 * kv_heads) * head_dim].view(T, kv_heads, head_dim)
        for t in range(T):
            p = int(positions[t])
            page = int(block_table[int(token_req[t]), p // page_size])
            k_plane[page, :, p % page_size] = k[t]
            v_plane[page, :, :, p % page_size] = v[t]


def paged_attention(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
                    tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale, splits=1, general=False, merge_tokens=None, waves=4):
    _attend(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
            tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale)


def _attend(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
            tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale):
    group = num_heads // num_kv_heads
    for tile in range(num_tiles):
        if tile_req is None:        # every request brings one token: tile i is the token of request i
            r, t0, first, n_new = tile, 0, tile, 1
        else:
            r = int(tile_req[tile]); t0 = int(tile_tok0[tile])
            first = int(req_indptr[r]); n_new = int(req_indptr[r + 1]) - first
        ctx = int(ctx_lens[r])
        for i in range(t0, min(t0 + tile_tokens, n_new)):
            pos = ctx + i
            lo = max(0, pos - window + 1) if window else 0
            keys = torch.arange(lo, pos + 1)
            pages = block_table[r, keys // page_size].long()
            k = k_plane[pages, :, keys % page_size].float()       # [n, kvh, hd]
            v = v_plane[pages, :, :, keys % page_size].float()
            qi = q[first + i].float().view(num_heads, head_dim)
            kk = k.repeat_interleave(group, dim=1)
            vv = v.repeat_interleave(group, dim=1)
            s = torch.einsum("hd,nhd->hn", qi, kk) * scale
            o = torch.einsum("hn,nhd->hd", torch.softmax(s, -1), vv)
            out[first + i] = o.reshape(-1).to(out.dtype)


def interleave_gate_up(gate, up):
    I, K = gate.shape
    blocks = -(-I // 32)
    g = torch.zeros((blocks * 32, K), dtype=gate.dtype)
    u = torch.zeros_like(g)
    g[:I] = gate
    u[:I] = up
    return torch.stack((g.view(blocks, 32, K), u.view(blocks, 32, K)), dim=1).reshape(blocks * 64, K).contiguous()


def linear_swiglu(x, gate_up, out):
    I, K = out.shape[1], x.shape[1]
    w = gate_up.float().view(-1, 2, 32, K)
    g = x.float() @ w[:, 0].reshape(-1, K)[:I].T
    u = x.float() @ w[:, 1].reshape(-1, K)[:I].T
    out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))


PREFILL_ATTENTION_ROWS = 64
PREFILL_ATTENTION_MAX_HEAD_DIM = 128


def prefill_attention_tile_tokens(num_heads, num_kv_heads):
    group = num_heads // num_kv_heads
    return max(1, PREFILL_ATTENTION_ROWS // min(group, ATTENTION_ROWS))


def paged_attention_prefill(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
                            tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale):
    _attend(q, out, k_plane, v_plane, block_table, req_indptr, ctx_lens, tile_req, tile_tok0, num_tiles,
            tile_tokens, num_heads, num_kv_heads, head_dim, page_size, window, scale)


def linear_partials_pay(M, N, K):
    return False


def linear_partials(x, weight):
    K = x.shape[1]
    half = (K // 2 // 8) * 8 or K
    a = x[:, :half].float() @ weight[:, :half].float().T
    b = x[:, half:].float() @ weight[:, half:].float().T
    return torch.stack((a, b))


def swiglu(gate_up, out):
    I = gate_up.shape[1] // 2
    g, u = gate_up[:, :I].float(), gate_up[:, I:].float()
    out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))


def _mix32(x):
    x = x & 0xFFFFFFFF
    x ^= x >> 16; x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15; x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def sample(logits, temperature, keys, out):
    for row in range(logits.shape[0]):
        t = float(temperature[row]) if temperature is not None else 0.0
        if t <= 0:
            out[row] = int(logits[row].argmax())
            continue
        key = int(keys[row]) & 0xFFFFFFFF
        best, besti = -math.inf, 0
        for i in range(logits.shape[1]):
            r = _mix32(_mix32(key ^ i) + 0x9E3779B9)
            u = ((r >> 8) + 0.5) / 16777216.0
            v = float(logits[row, i]) / t - math.log(-math.log(u))
            if v > best:
                best, besti = v, i
        out[row] = besti
