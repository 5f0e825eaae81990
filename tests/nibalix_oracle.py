"""Plain, slow Nibalix forward used as the ground truth of the tests.

One function per mechanism, written position by position in float64 from
the design's equations. It shares no code with the package: weights come
in as a ``{name: tensor}`` dict, the configuration as the plain dict that
``config.json`` holds, and every sequence is handled alone, from its first
token, with python loops over time.
"""

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean() + eps)


def norm_offset(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def canon(hs, w):
    """hs: list over time of [width]; w: [width, taps]. Returns h + conv(h)."""
    taps = w.shape[1]
    out = []
    for t in range(len(hs)):
        acc = hs[t].clone()
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                acc = acc + w[:, j] * hs[src]
        out.append(acc)
    return out


def rotate(v, pos, base, dims):
    """Rotate-half layout on the first ``dims`` entries of v."""
    out = v.clone()
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, w = v[i], v[i + half]
        out[i] = u * c - w * s
        out[i + half] = w * c + u * s
    return out


def latent_kv(hs, W, pre, mc, eps):
    """Per position: (latent c, rotated shared key part)."""
    r, rd = mc["kv_rank"], mc["rot_dim"]
    out = []
    for t, h in enumerate(hs):
        d = W[pre + "dkv"] @ h
        c = norm_plain(d[:r], W[pre + "dkv.norm"], eps)
        kr = rotate(d[r:r + rd], t, mc["rot"]["base"], mc["rot"]["dims"])
        out.append((c, kr))
    return out


def latent_attention(hs, kv, W, pre, mc):
    """hs: mixer inputs over time; kv: list of (c, k_rot) over time."""
    H, dn, rd, vd, r = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    win = (mc.get("mask") or {}).get("size")
    Wuk = W[pre + "uk"].view(H, dn, r)
    Wuv = W[pre + "uv"].view(H, vd, r)
    out = []
    for t, h in enumerate(hs):
        q = (W[pre + "q"] @ h).view(H, dn + rd)
        lo = 0 if win is None else max(0, t - win + 1)
        heads = []
        for hd in range(H):
            qn = q[hd, :dn]
            qr = rotate(q[hd, dn:], t, mc["rot"]["base"], mc["rot"]["dims"])
            sc = []
            for j in range(lo, t + 1):
                c, kr = kv[j]
                k = Wuk[hd] @ c
                sc.append((qn @ k + qr @ kr) * mc["scale"])
            p = torch.softmax(torch.stack(sc), 0)
            o = torch.zeros(vd, dtype=h.dtype)
            for n, j in enumerate(range(lo, t + 1)):
                o = o + p[n] * (Wuv[hd] @ kv[j][0])
            heads.append(o)
        out.append(W[pre + "o"] @ torch.cat(heads))
    return out


def mingru(hs, W, pre):
    n = W[pre + "z"].shape[0]
    S = torch.zeros(n, dtype=hs[0].dtype) if hs else None
    out = []
    for h in hs:
        z = torch.sigmoid(W[pre + "z"] @ h + W[pre + "z.b"])
        u = W[pre + "x"] @ h + W[pre + "x.b"]
        cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        S = (1 - z) * S + z * cand
        out.append(W[pre + "o"] @ (S * silu(W[pre + "g"] @ h)))
    return out


def moe(h, W, pre, fc):
    E, top = fc["router"]["experts"], fc["router"]["top"]
    z = W[pre + "router"] @ h + W[pre + "router.b"]
    val, idx = torch.topk(z, top)
    wts = torch.softmax(val, 0)
    out = torch.zeros_like(h)
    for k in range(top):
        e = int(idx[k])
        ep = f"{pre}e{e}."
        out = out + wts[k] * (W[ep + "down"] @ (silu(W[ep + "gate"] @ h) * (W[ep + "up"] @ h)))
    return out


def forward(cfg, W, tokens, dtype=F64, return_layers=False):
    """Logits [T, vocab] of one sequence (and the residual after every layer)."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    xs = [norm_offset(W["embed"][t], W["embed.norm"], eps) for t in tokens]
    kvs, layers_out = {}, []
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        hs = [norm_offset(x, W[p + "norm1"], eps) for x in xs]
        hm = canon(hs, W[p + "canon1"]) if cfg.get("canon") else hs
        mc = lc["mixer"]
        if lc["type"] == "latent_attention":
            src = mc.get("kv_from")
            if src is None:
                kvs[i] = latent_kv(hm, W, p + "mix.", mc, eps)
                src = i
            ys = latent_attention(hm, kvs[src], W, p + "mix.", mc)
        elif lc["type"] == "mingru":
            ys = mingru(hm, W, p + "mix.")
        else:
            raise ValueError(lc["type"])
        new = []
        for t, x in enumerate(xs):
            h = hs[t]
            acc = ys[t] * torch.sigmoid(W[p + "rg1"] @ h + W[p + "rg1.b"])
            if lc.get("mlp") is not None:
                acc = acc + moe(h, W, p + "mlp.", lc["mlp"]) * torch.sigmoid(
                    W[p + "rg2"] @ h + W[p + "rg2.b"])
            new.append(x + m * acc)
        xs = new
        layers_out.append(torch.stack(xs))
    logits = torch.stack([W["head"] @ norm_offset(x, W["final.norm"], eps) for x in xs])
    if return_layers:
        return logits, torch.stack(layers_out)
    return logits


# ---------------------------------------------------------------- fixtures

def random_weights(cfg, seed=0, scale=1.0):
    """Random bf16-representable weights with the design's tensor names."""
    g = torch.Generator().manual_seed(seed)

    def mat(o, i):
        return (torch.randn(o, i, generator=g) * scale / math.sqrt(i)).bfloat16().float()

    def vec(n, s=0.1):
        return (torch.randn(n, generator=g) * s).bfloat16().float()

    D = cfg["width"]
    W = {"embed": (torch.randn(cfg["vocab"], D, generator=g)).bfloat16().float(),
         "embed.norm": vec(D), "final.norm": vec(D), "head": mat(cfg["vocab"], D)}
    for i, lc in enumerate(cfg["layers"]):
        p, mc = f"l{i}.", lc["mixer"]
        W[p + "norm1"] = vec(D)
        if cfg.get("canon"):
            W[p + "canon1"] = (torch.randn(D, cfg["canon"]["taps"], generator=g) * 0.3).bfloat16().float()
        W[p + "rg1"], W[p + "rg1.b"] = mat(D, D), vec(D, 0.5)
        if lc["type"] == "latent_attention":
            H, dn, rd, vd, r = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
            W[p + "mix.q"] = mat(H * (dn + rd), D) * 2
            if mc.get("kv_from") is None:
                W[p + "mix.dkv"] = mat(r + rd, D)
                W[p + "mix.dkv.norm"] = 1.0 + vec(r)
            W[p + "mix.uk"], W[p + "mix.uv"] = mat(H * dn, r) * 2, mat(H * vd, r)
            W[p + "mix.o"] = mat(D, H * vd)
        else:
            n = mc["width"]
            W[p + "mix.z"], W[p + "mix.z.b"] = mat(n, D), vec(n, 0.5)
            W[p + "mix.x"], W[p + "mix.x.b"] = mat(n, D), vec(n, 0.5)
            W[p + "mix.g"], W[p + "mix.o"] = mat(n, D), mat(D, n)
        fc = lc.get("mlp")
        if fc is not None:
            W[p + "rg2"], W[p + "rg2.b"] = mat(D, D), vec(D, 0.5)
            E, ff = fc["router"]["experts"], fc["expert"]["ff"]
            W[p + "mlp.router"], W[p + "mlp.router.b"] = mat(E, D) * 2, vec(E, 0.5)
            for e in range(E):
                W[f"{p}mlp.e{e}.gate"], W[f"{p}mlp.e{e}.up"] = mat(ff, D), mat(ff, D)
                W[f"{p}mlp.e{e}.down"] = mat(D, ff)
    return {k: v.bfloat16().float() for k, v in W.items()}


def attn_layer(heads=2, dim=8, rot_dim=4, vdim=6, kv_rank=10, window=5, kv_from=None,
               base=100.0, scale=None, mlp=True, experts=3, top=2, ff=12, rot_dims=None):
    mc = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
          "mask": {"size": window}, "rot": {"base": base, "dims": rot_dims or rot_dim},
          "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim)}
    if kv_from is not None:
        mc["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mc, "mlp": moe_cfg(experts, top, ff) if mlp else None}


def gru_layer(width=24, mlp=True, experts=3, top=2, ff=12):
    return {"type": "mingru", "mixer": {"width": width},
            "mlp": moe_cfg(experts, top, ff) if mlp else None}


def moe_cfg(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_cfg(layers, width=16, vocab=40, taps=3, eps=1e-5, mult=0.5):
    return {"architecture": "Nibalix", "canon": {"taps": taps}, "layers": layers,
            "norm": {"eps": eps}, "residual_mult": mult, "vocab": vocab, "width": width}
