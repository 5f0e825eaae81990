"""Plain torch forms of the sequence-mixing ops (``ops/seqmix.py``).

They define the numerics of the HIP kernels in ``csrc_seqmix`` (each
kernel is tested against the function of the same name here) and are the
execution path of CPU runs. Everything the kernels keep in fp32 is fp32
here: norms, positions and angles, scores and softmax, recurrent state,
router logits and the residual sum.

Flat-batch conventions: a step holds ``T`` tokens of ``B`` sequences,
row ``b`` owning tokens ``cu[b]:cu[b+1]``; ``tok_seq[t]`` is the row of
token ``t``, ``positions[t]`` its position in its sequence, ``slots[b]``
the row's recurrent-state slot.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def offset_rmsnorm(x, w, eps, out_dtype):
    """x / sqrt(mean(x^2) + eps) * (1 + w) in fp32 -> (fp32, out_dtype)."""
    x = x.float()
    h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w.float())
    return h, h.to(out_dtype)


def causal_tap_conv(h, w, tails, cu, slots, out_dtype):
    """out_t = h_t + sum_j w[:, j] * h_(t - taps + 1 + j) per sequence, with
    the taps-1 inputs before the portion taken from ``tails[slot]``, which
    is then advanced to the portion's end. h fp32 [T, D]; w fp32 [D, taps];
    tails fp32 [slots, taps-1, D]."""
    taps = w.shape[1]
    out = torch.empty_like(h)
    cu_l, slots_l = cu.tolist(), slots.tolist()
    for b, s in enumerate(slots_l):
        a, e = cu_l[b], cu_l[b + 1]
        if e == a:
            continue
        ext = torch.cat([tails[s], h[a:e]], 0)          # [taps-1 + n, D]
        acc = h[a:e].clone()
        n = e - a
        for j in range(taps):
            acc += w[:, j] * ext[j:j + n]
        out[a:e] = acc
        if taps > 1:
            tails[s] = ext[ext.shape[0] - (taps - 1):]
    return out.to(out_dtype)


def _rotate_half(v, positions, base, dims):
    """Rotate the first ``dims`` entries of the last axis (fp32 in/out).
    v [T, ..., n]; positions [T]."""
    half = dims // 2
    i = torch.arange(half, device=v.device, dtype=torch.float32)
    freq = torch.exp2(i * (-2.0 / dims) * torch.log2(
        torch.tensor(float(base), device=v.device)))
    ang = positions.to(torch.float32)[:, None] * freq[None, :]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], -1)


def latent_prepare(proj, heads, dim, rot_dim, kv_rank, own_cache, norm_w, eps,
                   positions, rope_base, rope_dims, page_slot, cache):
    """From the packed [q | dkv] projection rows: write the normed latent
    and the rotated shared key part into ``cache`` rows ``page_slot``
    (layers with a cache of their own), and return the rotated query part
    [T, heads, rot_dim] in fp32."""
    T = proj.shape[0]
    q = proj[:, :heads * (dim + rot_dim)].view(T, heads, dim + rot_dim)
    q_rot = _rotate_half(q[..., dim:].float(), positions, rope_base, rope_dims)
    if own_cache:
        d = proj[:, heads * (dim + rot_dim):].float()
        c = d[:, :kv_rank]
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
        kr = _rotate_half(d[:, kv_rank:kv_rank + rot_dim], positions,
                          rope_base, rope_dims)
        cache[page_slot.long()] = torch.cat([c, kr], -1).to(cache.dtype)
    return q_rot


def latent_window_attention(q_lat, q_rot, cache, kv_rank, block_tables,
                            block_size, cu, positions, window, scale,
                            out_dtype):
    """Softmax attention in latent space over a paged cache.

    q_lat [H, T, kv_rank] (the query already folded through the key
    up-projection), q_rot fp32 [T, H, rot_dim], cache rows
    [c (kv_rank) | k_rot]. Token at position p sees positions j with
    0 <= p - j < window (window 0: all j <= p). Returns sum_j p_j c_j,
    [H, T, kv_rank]."""
    H, T, r = q_lat.shape
    out = torch.zeros(H, T, r, dtype=torch.float32, device=q_lat.device)
    cu_l = cu.tolist()
    pos_l = positions.tolist()
    for b in range(len(cu_l) - 1):
        a, e = cu_l[b], cu_l[b + 1]
        if e == a:
            continue
        p0, p1 = pos_l[a], pos_l[e - 1]
        lo = 0 if window <= 0 else max(0, p0 - window + 1)
        j = torch.arange(lo, p1 + 1, device=cache.device)
        rows = block_tables[b].long()[j // block_size] * block_size + j % block_size
        kv = cache[rows].float()
        c, kr = kv[:, :kv_rank], kv[:, kv_rank:]
        s = torch.einsum("htr,jr->htj", q_lat[:, a:e].float(), c)
        s = s + torch.einsum("thd,jd->htj", q_rot[a:e].float(), kr)
        s = s * scale
        p = positions[a:e].long()[:, None]
        ok = j[None, :] <= p
        if window > 0:
            ok = ok & (p - j[None, :] < window)
        s = s.masked_fill(~ok[None], float("-inf"))
        out[:, a:e] = torch.einsum("htj,jr->htr", torch.softmax(s, -1), c)
    return out.to(out_dtype)


def mingru_scan(zxg, bias, state, cu, slots, out_dtype):
    """zxg [T, 3n] = [z | x | g] pre-activations (bias [3n] fp32 still to
    add); state fp32 [slots, n], advanced in place. Returns S_t * silu(g_t)."""
    n = zxg.shape[1] // 3
    v = zxg.float() + bias.float()
    z = torch.sigmoid(v[:, :n])
    u = v[:, n:2 * n]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = v[:, 2 * n:]
    gate = g * torch.sigmoid(g)
    out = torch.empty(zxg.shape[0], n, dtype=torch.float32, device=zxg.device)
    cu_l, slots_l = cu.tolist(), slots.tolist()
    for b, s in enumerate(slots_l):
        S = state[s]
        for t in range(cu_l[b], cu_l[b + 1]):
            S = (1.0 - z[t]) * S + z[t] * cand[t]
            out[t] = S * gate[t]
        state[s] = S
    return out.to(out_dtype)


def moe_route(h, router_w, router_b, top):
    """fp32 router: logits = W h + b; the ``top`` largest (ties: lowest
    index first); weights = softmax over the chosen logits."""
    z = F.linear(h.float(), router_w.float(), router_b.float())
    val, idx = torch.sort(z, dim=-1, descending=True, stable=True)
    val, idx = val[:, :top], idx[:, :top]
    return idx.to(torch.int32), torch.softmax(val, -1)


def moe_experts(h, idx, wts, exp_gu, exp_down):
    """sum_k wts[t,k] * down_e(silu(gate_e h) * up_e h), e = idx[t,k].
    exp_gu [E, 2ff, D] = per expert [gate; up]; exp_down [E, D, ff].
    Returns fp32 [T, D]."""
    T, D = h.shape
    E, ff2, _ = exp_gu.shape
    ff = ff2 // 2
    out = torch.zeros(T, D, dtype=torch.float32, device=h.device)
    for e in range(E):
        hit = idx == e
        rows = hit.any(-1).nonzero().flatten()
        if rows.numel() == 0:
            continue
        gu = F.linear(h[rows], exp_gu[e])
        g = gu[:, :ff].float()
        act = (g * torch.sigmoid(g) * gu[:, ff:].float()).to(h.dtype)
        y = F.linear(act, exp_down[e]).float()
        w = (wts[rows] * hit[rows]).sum(-1, keepdim=True)
        out[rows] += w * y
    return out


def gated_residual_add(x, mix, ff, gates, gate_b, mult):
    """x += mult * (mix * sigmoid(g1) + ff * sigmoid(g2)) on the fp32
    residual, in place. gates [T, D or 2D] pre-bias; ff None when the
    layer has no feed-forward."""
    D = x.shape[1]
    g = torch.sigmoid(gates.float() + gate_b.float())
    acc = mix.float() * g[:, :D]
    if ff is not None:
        acc = acc + ff.float() * g[:, D:2 * D]
    x.add_(acc, alpha=mult)
    return x
