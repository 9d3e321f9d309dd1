"""Plain PyTorch counterparts of the HIP kernels, one function per kernel, with the
same call signatures as ``yalis_amd.ops.hip.HipOps``.

Two uses: the GPU tests compare each kernel with its counterpart here at sizes of
their own; and ``RefOps`` lets the CPU tests run the framework's host logic (batching,
paging, scheduling) without a GPU.  It is test equipment: the framework never imports
it.  Everything is computed in float32 and rounded once to the output dtype.
"""
from __future__ import annotations

import math

import torch


def embed(token_ids, table):
    return table[token_ids.long()].to(torch.float32)


def add_rmsnorm(residual, delta, weight, eps, unit_offset, out_dtype):
    """residual += delta in place (float32); returns the normalised rows."""
    if delta is not None:
        residual += delta.to(torch.float32)
    return _rmsnorm(residual, weight, eps, unit_offset).to(out_dtype)


def gather_add_rmsnorm(residual, delta, rows, weight, eps, unit_offset, out_dtype):
    v = residual[rows.long()]
    if delta is not None:
        v = v + delta[rows.long()].to(torch.float32)
    return _rmsnorm(v, weight, eps, unit_offset).to(out_dtype)


def _rmsnorm(x, weight, eps, unit_offset):
    ms = (x * x).mean(dim=-1, keepdim=True)
    w = weight.to(torch.float32)
    if unit_offset:
        w = w + 1.0
    return x * torch.rsqrt(ms + eps) * w


def rmsnorm(x, weight, eps, unit_offset, out_dtype):
    """The norm of rows that are no residual stream."""
    return _rmsnorm(x.to(torch.float32), weight, eps, unit_offset).to(out_dtype)


def linear(x, w, out_dtype, partial_ok=False, bias=None):
    y = x.to(torch.float32) @ w.to(torch.float32).T
    if bias is not None:  # added to the float32 product, one rounding (torch's addmm, the reference's biased Linear)
        y = y + bias.to(torch.float32)
    return y.to(out_dtype)


def rope_append(qkv, n_heads, n_kv, head_dim, positions, cos, sin, rotary_dim, interleaved,
                k_cache, v_cache, slots, page_size):
    """Rotates the query heads of ``qkv`` in place; rotates the key heads and stores
    them, and the value heads transposed, at each token's slot of the pages.  Returns the
    tensor whose rows start with the rotated queries."""
    n = qkv.shape[0]
    x = qkv.view(n, n_heads + 2 * n_kv, head_dim)
    rot = x[:, : n_heads + n_kv].to(torch.float32)
    if rotary_dim:
        c = cos[positions.long()][:, None, :]
        s = sin[positions.long()][:, None, :]
        if interleaved:
            a = rot[..., 0:rotary_dim:2]
            b = rot[..., 1:rotary_dim:2]
        else:
            a = rot[..., : rotary_dim // 2]
            b = rot[..., rotary_dim // 2 : rotary_dim]
        ra = a * c - b * s
        rb = b * c + a * s
        rot = rot.clone()
        if interleaved:
            rot[..., 0:rotary_dim:2] = ra
            rot[..., 1:rotary_dim:2] = rb
        else:
            rot[..., : rotary_dim // 2] = ra
            rot[..., rotary_dim // 2 : rotary_dim] = rb
    rot = rot.to(qkv.dtype)
    x[:, :n_heads] = rot[:, :n_heads]
    if n_kv:
        page = (slots // page_size).long()
        off = (slots % page_size).long()
        k_cache[page, :, off, :] = rot[:, n_heads:]
        v_cache[page, :, :, off] = x[:, n_heads + n_kv :]
    return qkv


def attention_paged(q, k_cache, v_cache, positions, token_seq, block_table, page_size, scale, window):
    """q: [N, H, D]; pages as in the framework (keys [pages, G, page, D], values
    [pages, G, D, page]).  Gathers each token's visible keys through its request's
    block table and runs a float32 softmax."""
    n, n_heads, d = q.shape
    n_kv = k_cache.shape[1]
    qpk = n_heads // n_kv
    out = torch.empty((n, n_heads, d), dtype=torch.float32, device=q.device)
    for t in range(n):
        pos = int(positions[t])
        lo = max(0, pos - window + 1) if window else 0
        keys = torch.arange(lo, pos + 1, device=q.device)
        pages = block_table[int(token_seq[t])][(keys // page_size).long()].long()
        offs = (keys % page_size).long()
        k = k_cache[pages, :, offs, :].to(torch.float32)  # [keys, G, D]
        v = v_cache[pages, :, :, offs].to(torch.float32)  # [keys, G, D]
        for h in range(n_heads):
            g = h // qpk
            s = (k[:, g, :] @ q[t, h].to(torch.float32)) * scale
            p = torch.softmax(s, dim=0)
            out[t, h] = p @ v[:, g, :]
    return out


def attention(qkv, n_heads, n_kv, head_dim, k_cache, v_cache, page_size, scale,
              window, ctx, group, tiles, long_tiles=None, plan=None, long_plan=None, long_col_tiles=1, token_cols=None):
    n = qkv.shape[0]
    q = qkv.view(n, -1, head_dim)[:, :n_heads]
    out = attention_paged(
        q, k_cache, v_cache, ctx.arrays["positions"], ctx.arrays["token_seq"],
        ctx.arrays[f"block_table_g{group}"], page_size, scale, window,
    )
    return out.reshape(n, n_heads * head_dim).to(qkv.dtype)


def gated_act(gu, activation, out_dtype=None, group=0):
    inter = gu.shape[1] // 2
    if group:
        pairs = gu.reshape(gu.shape[0], inter // group, 2, group)
        g = pairs[:, :, 0, :].reshape(gu.shape[0], inter).to(torch.float32)
        u = pairs[:, :, 1, :].reshape(gu.shape[0], inter).to(torch.float32)
    else:
        g = gu[:, :inter].to(torch.float32)
        u = gu[:, inter:].to(torch.float32)
    if activation == "silu":
        a = g * torch.sigmoid(g)
    elif activation == "gelu_tanh":
        a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g**3)))
    else:
        raise ValueError(activation)
    return (a * u).to(out_dtype or gu.dtype)


def argmax(logits):
    return torch.argmax(logits, dim=-1).to(torch.int32)


class RefOps:
    """The kernel library's interface over the functions above (CPU or GPU tensors)."""

    def check_attention_sizes(self, n_heads, n_kv, head_dim, page_size):
        assert n_heads % n_kv == 0 and head_dim % 16 == 0 and page_size % 16 == 0

    def attention_tokens_per_tile(self, n_heads, n_kv):
        return 16 // min(n_heads // n_kv, 16)

    def attention_long_span_tile(self, n_heads, n_kv, col_tiles=1):
        return 4 * col_tiles * self.attention_tokens_per_tile(n_heads, n_kv)

    @staticmethod
    def attention_long_col_tiles(workgroups, fewest_keys):
        return 1

    embed = staticmethod(embed)
    add_rmsnorm = staticmethod(add_rmsnorm)
    gather_add_rmsnorm = staticmethod(gather_add_rmsnorm)
    rmsnorm = staticmethod(rmsnorm)
    linear = staticmethod(linear)
    rope_append = staticmethod(rope_append)
    attention = staticmethod(attention)
    gated_act = staticmethod(gated_act)
    argmax = staticmethod(argmax)

    @staticmethod
    def pack_gate_up(w_gate, w_up):
        return torch.cat([w_gate, w_up], dim=0).contiguous(), 0

    @staticmethod
    def gate_up_act(x, w_gate_up, group, activation, out_dtype):
        return gated_act(linear(x, w_gate_up, out_dtype), activation, out_dtype, group)

    def sample(self, logits, temperature, top_k, top_p, seeds, draws, whole_row=False):
        from plain_llama import sample_token

        out = []
        for i in range(logits.shape[0]):
            k = int(top_k[i])
            out.append(
                sample_token(logits[i].cpu(), float(temperature[i]), k if k > 0 else None, float(top_p[i]), int(seeds[i]), int(draws[i]))
            )
        return torch.tensor(out, dtype=torch.int32, device=logits.device)


# ------------------------------------------------------------------ tiled cache pages
# The matrix-core attention keeps bfloat16 pages of a multiple of 64 tokens (head sizes 64 and
# 128) in the order its loads take them.  Written out here once more, from the layout's
# description (yalis_amd/csrc/common.h), so that tests can fill pages and read them back:
#   keys:   within a block of 64 slots, piece (((u*2 + sb) * D/32 + ks) * 4 + g) * 16 + r holds
#           dims 32ks + 8g .. +7 of slot 32u + 8(r/4) + 4sb + r%4;
#   values: piece ((u * D/16 + dt) * 4 + g) * 16 + r holds slots 32u + 8g .. +7 of dim 16dt + r.
def _tiled_indices(page, d):
    import numpy as np

    slot = np.arange(page)[:, None]
    dim = np.arange(d)[None, :]
    j = slot % 64
    u, a, sb, b = j // 32, (j % 32) // 8, (j % 8) // 4, j % 4
    piece_k = (((u * 2 + sb) * (d // 32) + dim // 32) * 4 + (dim % 32) // 8) * 16 + 4 * a + b
    k_at = (slot // 64) * 64 * d + piece_k * 8 + dim % 8            # [slot, dim] -> offset in the slab
    piece_v = ((u * (d // 16) + dim // 16) * 4 + (j % 32) // 8) * 16 + dim % 16
    v_at = (slot // 64) * 64 * d + piece_v * 8 + j % 8              # [slot, dim] -> offset in the slab
    assert sorted(k_at.ravel()) == list(range(page * d)) and sorted(v_at.ravel()) == list(range(page * d))
    return torch.from_numpy(k_at.ravel()), torch.from_numpy(v_at.T.copy().ravel())  # in the plain slabs' element order


def tile_cache(k_plain, v_plain):
    """Plain pages ([pages, kv, page, D] keys, [pages, kv, D, page] values) -> the same shapes
    holding the tiled order."""
    n, g, page, d = k_plain.shape
    k_at, v_at = _tiled_indices(page, d)
    k = torch.empty_like(k_plain).view(n, g, page * d)
    v = torch.empty_like(v_plain).view(n, g, page * d)
    k[:, :, k_at] = k_plain.reshape(n, g, page * d)
    v[:, :, v_at] = v_plain.reshape(n, g, page * d)
    return k.view(n, g, page, d), v.view(n, g, d, page)


def untile_cache(k_tiled, v_tiled):
    n, g, page, d = k_tiled.shape
    k_at, v_at = _tiled_indices(page, d)
    k = k_tiled.reshape(n, g, page * d)[:, :, k_at]
    v = v_tiled.reshape(n, g, page * d)[:, :, v_at]
    return k.reshape(n, g, page, d), v.reshape(n, g, d, page)
