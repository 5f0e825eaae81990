"""Plain, slow Nedasun forward used as the ground truth of the tests.

One function per mechanism, written position by position in float64 from
the design's equations. It shares no code with the package: weights come
in as a ``{name: tensor}`` dict, the configuration as the plain dict that
``config.json`` holds, and every sequence is handled alone, from its first
token, with python loops over time.
"""

import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------ norms

def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean() + eps)


def norm_offset(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


# -------------------------------------------------------------- attention

def rotate_pairs(v, pos, base, dims):
    """Interleaved layout: entries (2i, 2i+1) of the first ``dims`` form a
    pair; the rest pass through."""
    out = v.clone()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, w = v[2 * i], v[2 * i + 1]
        out[2 * i] = u * c - w * s
        out[2 * i + 1] = w * c + u * s
    return out


def attention_values(hs, W, pre, mc, v_first):
    """Per position the [G, vdim] values, after mixing with the first
    value-mixing layer's values when ``v_first`` is given."""
    G, vd = mc["kv_heads"], mc["vdim"]
    out = []
    for t, h in enumerate(hs):
        v = (W[pre + "v"] @ h).view(G, vd)
        if v_first is not None:
            lam = W[pre + "vmix"]
            v = (1.0 - lam) * v + lam * v_first[t]
        out.append(v)
    return out


def attention(hs, W, pre, mc, values):
    """Softmax attention with capped scores, a per-head sink in the
    denominator, and head mixing of the weights. ``values``: per position
    [G, vdim] (already value-mixed)."""
    H, G, dk, vd = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    rot = mc.get("rot") or {}
    base, dims = rot.get("base", 10000.0), rot.get("dims", 0)
    cap, scale = mc.get("softcap"), mc["scale"]
    rep = H // G
    qs, ks = [], []
    for t, h in enumerate(hs):
        q = (W[pre + "q"] @ h).view(H, dk)
        k = (W[pre + "k"] @ h).view(G, dk)
        qs.append(torch.stack([rotate_pairs(q[i], t, base, dims) for i in range(H)]))
        ks.append(torch.stack([rotate_pairs(k[i], t, base, dims) for i in range(G)]))
    talk = W.get(pre + "talk")
    out = []
    for t in range(len(hs)):
        wts = torch.zeros(H, t + 1, dtype=F64)
        for hd in range(H):
            s = torch.stack([(qs[t][hd] * ks[j][hd // rep]).sum() * scale
                             for j in range(t + 1)])
            if cap:
                s = cap * torch.tanh(s / cap)
            sink = W[pre + "sink"][hd] if pre + "sink" in W else None
            m = s.max() if sink is None else torch.maximum(s.max(), sink)
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink - m) if sink is not None else 0.0)
            wts[hd] = e / den
        if talk is not None:
            wts = talk @ wts
        o = torch.zeros(H, vd, dtype=F64)
        for hd in range(H):
            for j in range(t + 1):
                o[hd] += wts[hd, j] * values[j][hd // rep]
        out.append(W[pre + "o"] @ o.reshape(-1))
    return out


# ------------------------------------------------------------- delta rule

def short_conv_silu(xs, w):
    """xs: list over time of [channels]; w [channels, taps], the last
    column multiplying the current token; zeros before the start."""
    taps = w.shape[1]
    out = []
    for t in range(len(xs)):
        acc = torch.zeros_like(xs[t])
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                acc = acc + w[:, j] * xs[src]
        out.append(silu(acc))
    return out


def delta_mixer(hs, W, pre, mc, eps):
    H, G, dk, vd = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    rep = H // G
    q = short_conv_silu([W[pre + "q"] @ h for h in hs], W[pre + "q.conv"])
    k = short_conv_silu([W[pre + "k"] @ h for h in hs], W[pre + "k.conv"])
    v = short_conv_silu([W[pre + "v"] @ h for h in hs], W[pre + "v.conv"])
    S = [torch.zeros(dk, vd, dtype=F64) for _ in range(H)]
    out = []
    for t, h in enumerate(hs):
        qt, kt, vt = q[t].view(G, dk), k[t].view(G, dk), v[t].view(H, vd)
        beta = torch.sigmoid(W[pre + "b"] @ h)
        step = torch.nn.functional.softplus(W[pre + "a"] @ h + W[pre + "dt_bias"])
        decay = torch.exp(-torch.exp(W[pre + "A_log"]) * step)
        gate = silu(W[pre + "g"] @ h).view(H, vd)
        o = torch.zeros(H, vd, dtype=F64)
        for hd in range(H):
            qq, kk = qt[hd // rep], kt[hd // rep]
            qq = qq / torch.sqrt((qq * qq).sum() + 1e-6) * dk ** -0.5
            kk = kk / torch.sqrt((kk * kk).sum() + 1e-6)
            S[hd] = decay[hd] * S[hd]
            u = beta[hd] * (vt[hd] - S[hd].T @ kk)
            S[hd] = S[hd] + torch.outer(kk, u)
            r = S[hd].T @ qq
            o[hd] = unit_rms(r, eps) * W[pre + "norm"] * gate[hd]
        out.append(W[pre + "o"] @ o.reshape(-1))
    return out


# ----------------------------------------------------------- feed-forward

def capped_glu(h, W, pre, limit):
    g = torch.clamp(W[pre + "gate"] @ h, max=limit)
    u = torch.clamp(W[pre + "up"] @ h, min=-limit, max=limit)
    return W[pre + "down"] @ (g * torch.sigmoid(1.702 * g) * (u + 1.0))


def moe(h, W, pre, fc):
    rc = fc["router"]
    E, ident, top = rc["experts"], rc.get("identity", 0), rc["top"]
    s = torch.softmax(W[pre + "router"] @ h, 0)
    choice = s + W[pre + "correction"] if pre + "correction" in W else s
    picked = torch.topk(choice, top).indices.tolist()
    y = torch.zeros_like(h)
    for e in picked:
        w = s[e] * rc.get("scale", 1.0)
        if e >= E:
            assert e < E + ident
            y = y + w * h
        else:
            y = y + w * capped_glu(h, W, f"{pre}e{e}.", fc["expert"]["limit"])
    if fc.get("shared"):
        y = y + capped_glu(h, W, pre + "shared.", fc["shared"]["limit"])
    return y


def feed_forward(h, W, pre, fc):
    if fc["kind"] == "dense":
        return capped_glu(h, W, pre, fc["limit"])
    return moe(h, W, pre, fc)


# ------------------------------------------------------------------ model

def forward(cfg, W, tokens):
    """Logits [T, vocab] and the residual stream after every layer
    [layers, T, width] of one sequence from its first token (float64)."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    xs = [W["embed"][t].clone() for t in tokens]
    v_first = None
    stream = []
    for i, lc in enumerate(cfg["layers"]):
        p, mc = f"l{i}.", lc["mixer"]
        hs = [norm_offset(x, W[p + "norm1"], eps) for x in xs]
        if lc["type"] == "attention":
            mixes = bool(mc.get("v_mix"))
            vals = attention_values(hs, W, p + "mix.", mc,
                                    v_first if mixes else None)
            if mixes and v_first is None:
                v_first = vals
            ys = attention(hs, W, p + "mix.", mc, vals)
        elif lc["type"] == "delta":
            ys = delta_mixer(hs, W, p + "mix.", mc, eps)
        else:
            raise ValueError(lc["type"])
        xs = [x + norm_offset(y, W[p + "norm1b"], eps) for x, y in zip(xs, ys)]
        if lc.get("mlp") is not None:
            for t, x in enumerate(xs):
                h = norm_offset(x, W[p + "norm2"], eps)
                f = feed_forward(h, W, p + "mlp.", lc["mlp"])
                xs[t] = x + norm_offset(f, W[p + "norm2b"], eps)
        stream.append(torch.stack(xs))
    logits = torch.stack([W["head"] @ norm_offset(x, W["final.norm"], eps) for x in xs])
    return logits, torch.stack(stream)


# ---------------------------------------------------------- random models

def tensor_shapes(cfg):
    """{tensor name: shape} of a configuration."""
    D = cfg["width"]
    out = {"embed": (cfg["vocab"], D), "final.norm": (D,), "head": (cfg["vocab"], D)}

    def glu(pre, ff):
        out[pre + "gate"], out[pre + "up"], out[pre + "down"] = (ff, D), (ff, D), (D, ff)

    for i, lc in enumerate(cfg["layers"]):
        p, mc = f"l{i}.", lc["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (D,)
        H, G, dk, vd = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        m = p + "mix."
        if lc["type"] == "attention":
            out[m + "q"], out[m + "k"], out[m + "v"] = (H * dk, D), (G * dk, D), (G * vd, D)
            out[m + "vmix"], out[m + "talk"], out[m + "sink"] = (), (H, H), (H,)
        else:
            taps = mc["conv"]
            out[m + "q"], out[m + "k"], out[m + "v"] = (G * dk, D), (G * dk, D), (H * vd, D)
            out[m + "q.conv"], out[m + "k.conv"] = (G * dk, taps), (G * dk, taps)
            out[m + "v.conv"] = (H * vd, taps)
            out[m + "b"], out[m + "a"] = (H, D), (H, D)
            out[m + "A_log"], out[m + "dt_bias"] = (H,), (H,)
            out[m + "norm"], out[m + "g"] = (vd,), (H * vd, D)
        out[m + "o"] = (D, H * vd)
        fc = lc.get("mlp")
        if fc is None:
            continue
        out[p + "norm2"] = out[p + "norm2b"] = (D,)
        f = p + "mlp."
        if fc["kind"] == "dense":
            glu(f, fc["ff"])
        else:
            rc = fc["router"]
            n = rc["experts"] + rc.get("identity", 0)
            out[f + "router"], out[f + "correction"] = (n, D), (n,)
            for e in range(rc["experts"]):
                glu(f"{f}e{e}.", fc["expert"]["ff"])
            if fc.get("shared"):
                glu(f + "shared.", fc["shared"]["ff"])
    return out


def random_weights(cfg, seed=0, round_bf16=True):
    """Random weights at magnitudes that keep every mechanism visible:
    sinks, head mixing, value mixing, decays and the router correction all
    move the output by more than rounding."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, shape in tensor_shapes(cfg).items():
        r = torch.randn(shape, generator=g, dtype=torch.float32)
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            pass
        elif last == "talk":
            r = torch.eye(shape[0]) + 0.3 * r
        elif last == "vmix":
            r = 0.3 + 0.1 * r
        elif last == "conv":
            r = 0.5 * r
        elif last == "norm" and name != "final.norm":
            r = 1.0 + 0.1 * r
        elif last == "correction":
            r = 0.05 * r
        elif last == "router":
            r = 2.0 * r / math.sqrt(shape[-1])
        elif len(shape) >= 2:
            r = 1.5 * r / math.sqrt(shape[-1])
        elif last in ("sink", "A_log", "dt_bias"):
            r = 0.5 * r
        else:
            r = 0.1 * r
        W[name] = r.to(torch.bfloat16).float() if round_bf16 else r
    return W


# ------------------------------------------------------- config builders

def attn_layer(heads=4, kv_heads=2, dim=8, vdim=6, rot_dims=None, base=10000.0,
               scale=None, softcap=5.0, v_mix=True, mlp="dense"):
    mc = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
          "scale": dim ** -0.5 if scale is None else scale, "softcap": softcap,
          "rot": {"base": base, "dims": dim if rot_dims is None else rot_dims},
          "v_mix": v_mix}
    return {"type": "attention", "mixer": mc, "mlp": mlp_cfg(mlp)}


def delta_layer(heads=4, kv_heads=2, dim=8, vdim=6, conv=3, mlp="moe"):
    mc = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}
    return {"type": "delta", "mixer": mc, "mlp": mlp_cfg(mlp)}


def mlp_cfg(kind, **kw):
    if kind is None or isinstance(kind, dict):
        return kind
    if kind == "dense":
        return {"kind": "dense", "ff": kw.get("ff", 24), "limit": kw.get("limit", 0.8)}
    return {"kind": "moe",
            "expert": {"ff": kw.get("ff", 10), "limit": kw.get("limit", 0.6)},
            "router": {"experts": kw.get("experts", 5), "identity": kw.get("identity", 1),
                       "scale": kw.get("scale", 1.7), "top": kw.get("top", 2)},
            "shared": ({"ff": kw.get("shared_ff", 12), "limit": kw.get("shared_limit", 0.9)}
                       if kw.get("shared", True) else None)}


def make_cfg(layers, width=16, vocab=41, eps=1e-5):
    return {"architecture": "Nedasun", "layers": layers, "norm": {"eps": eps},
            "vocab": vocab, "width": width}
