"""Nedasun (sandwich-block layer-list model) against the plain oracle in
nedasun_oracle.py.

Every test builds its own small configuration and random weights. The
``dev`` fixture runs each case on the CPU path and, marked ``gpu``, on the
HIP kernels (fp32 and bf16 models).
"""

import json
import math
import os
import subprocess
import sys

import pytest
import torch

import nedasun_oracle as O
from distrl_llm_amd.config import EngineConfig, SamplingParams
from distrl_llm_amd.engine.hybrid_engine import HybridEngine
from distrl_llm_amd.models.hybrid import (HybridLM, nedasun_spec_from_config,
                                          save_nedasun_checkpoint)
from distrl_llm_amd.ops import seqmix as SM

CASES = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
         pytest.param(("cuda", torch.float32), id="gpu-f32", marks=pytest.mark.gpu),
         pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu)]


@pytest.fixture(params=CASES)
def dev(request):
    return request.param


def tol(dtype):
    # bf16 is a coarse check here: seven layers only 16 wide, and a router
    # choice may flip on a rounding. The same kernels are held to 2e-4 in
    # fp32, and the bf16-only tiled attention kernel has a test of its own.
    return 2e-4 if dtype == torch.float32 else 0.15


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    return float(d.pow(2).mean().sqrt() / want.pow(2).mean().sqrt().clamp_min(1e-9))


def mixed_cfg():
    """Sizes that differ from one another wherever the design allows it: the
    first attention layer mixes no values, the first mixing layer is not
    layer 0, heads/kv_heads ratios 1, 2 and 3, partial and no rotation, key
    dims that do not fill a lane's 32 state rows or spill into a second
    lane, and every feed-forward form."""
    return O.make_cfg([
        O.attn_layer(heads=2, kv_heads=2, dim=6, vdim=5, rot_dims=4, v_mix=False, softcap=0.0,
                     mlp=O.mlp_cfg("moe", experts=3, identity=0, top=1, shared=False)),
        O.delta_layer(heads=4, kv_heads=2, dim=8, vdim=6, conv=3, mlp="dense"),
        O.attn_layer(heads=6, kv_heads=2, dim=8, vdim=7, rot_dims=8, scale=0.31, softcap=3.0,
                     mlp=O.mlp_cfg("moe", experts=4, identity=2, top=3)),
        O.delta_layer(heads=3, kv_heads=1, dim=40, vdim=5, conv=4, mlp=None),
        O.attn_layer(heads=6, kv_heads=2, dim=10, vdim=7, rot_dims=0, softcap=8.0, mlp=None),
        O.delta_layer(heads=2, kv_heads=2, dim=5, vdim=70, conv=1,
                      mlp=O.mlp_cfg("moe", experts=2, identity=1, top=3, scale=0.9)),
        O.attn_layer(heads=3, kv_heads=1, dim=8, vdim=14, rot_dims=6, base=77.0, v_mix=False,
                     mlp="dense"),
    ], width=16, vocab=37)


def build(cfg, dev, seed=0, blocks=64, block_size=4, slots=4, W=None):
    device, dtype = dev
    W = W if W is not None else O.random_weights(cfg, seed)
    model = HybridLM(nedasun_spec_from_config(cfg), dtype=dtype, device=device)
    model.load_tensors(W)
    eng = HybridEngine(model, EngineConfig(max_seq_length=4096, kv_block_size=block_size,
                                           num_kv_blocks=blocks, num_state_slots=slots,
                                           max_num_seqs=slots), device=torch.device(device))
    return W, eng


def run_portions(eng, tokens, cuts, capture=None):
    q = eng.open_sequence()
    out, at = [], 0
    for n in cuts:
        out.append(eng.step([(q, tokens[at:at + n])], [list(range(n))], capture=capture))
        at += n
    assert at == len(tokens)
    eng.close_sequence(q)
    return torch.cat(out)


def toks(n, vocab, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def ints(v, device):
    return torch.tensor(v, dtype=torch.int32, device=device)


# ------------------------------------------------------ mechanisms alone

def test_sandwich_residual_norm(dev):
    device, dtype = dev
    g = torch.Generator().manual_seed(0)
    T, D, eps = 5, 24, 1e-5
    x = torch.randn(T, D, generator=g)
    y = torch.randn(T, D, generator=g).to(dtype).float()
    y2 = torch.randn(T, D, generator=g)
    pw, nw = 0.2 * torch.randn(D, generator=g), 0.2 * torch.randn(D, generator=g)
    for second in (None, y2):
        xd = x.clone().to(device)
        h = SM.sandwich_residual_norm(xd, y.to(dtype).to(device),
                                      None if second is None else second.to(device),
                                      pw.to(device), nw.to(device), eps, dtype)
        s = y.double() if second is None else y.double() + second.double()
        want_x = torch.stack([x[t].double() + O.norm_offset(s[t], pw.double(), eps) for t in range(T)])
        want_h = torch.stack([O.norm_offset(want_x[t], nw.double(), eps) for t in range(T)])
        assert rel_err(xd, want_x) < 1e-6
        assert rel_err(h, want_h) < (1e-6 if dtype == torch.float32 else 5e-3)
        assert SM.sandwich_residual_norm(xd, y.to(dtype).to(device), None, pw.to(device), None,
                                         eps, dtype) is None


def test_pair_rotation_value_blend_and_cache_rows(dev):
    device, dtype = dev
    H, G, dk, vd, dims, base = 4, 2, 8, 5, 6, 300.0
    g = torch.Generator().manual_seed(1)
    T = 6
    proj = torch.randn(T, H * dk + G * dk + G * vd, generator=g).to(dtype)
    vf = torch.randn(T, G * vd + 3, generator=g).to(dtype)[:, 3:]      # a strided view
    pos = [0, 1, 2, 700, 3, 4]
    slot = [9, 2, 5, 0, 7, 11]
    cache = torch.full((12, G * (dk + vd)), 7.0, dtype=dtype, device=device)
    lam = torch.tensor([0.3])
    q = SM.rope_kv_write(proj.to(device), H, G, dk, vd, ints(pos, device), base, dims,
                         ints(slot, device), cache, lam.to(device), vf.to(device))
    t = 3e-5 if dtype == torch.float32 else 8e-3     # fp32 angles at position 700
    for i in range(T):
        for hd in range(H):
            want = O.rotate_pairs(proj[i, hd * dk:(hd + 1) * dk].double(), pos[i], base, dims)
            assert rel_err(q[i, hd], want) < t
        for c in range(G):
            a = H * dk + c * dk
            want = O.rotate_pairs(proj[i, a:a + dk].double(), pos[i], base, dims)
            assert rel_err(cache[slot[i], c * dk:(c + 1) * dk], want) < t
        v = proj[i, (H + G) * dk:].double()
        assert rel_err(cache[slot[i], G * dk:], 0.7 * v + 0.3 * vf[i].double()) < t
    untouched = [r for r in range(12) if r not in slot]
    assert bool((cache[untouched].float() == 7.0).all())
    # without a first layer the values pass unblended
    SM.rope_kv_write(proj.to(device), H, G, dk, vd, ints(pos, device), base, dims,
                     ints(slot, device), cache, lam.to(device), None)
    assert rel_err(cache[slot[0], G * dk:], proj[0, (H + G) * dk:].double()) < t


def _attend(dev, H, G, dk, vd, bs, table, pos, cache, q, scale=1.0, softcap=0.0, sink=None,
            talk=None, rows=None):
    device, dtype = dev
    n = len(pos)
    rows = rows if rows is not None else [(0, n)]
    cu, seq = [0], []
    for b, (_, cnt) in enumerate(rows):
        cu.append(cu[-1] + cnt)
        seq += [b] * cnt
    tiles, mt = SM.query_tiles([c for _, c in rows], SM.WIDE_QUERY_TILE)
    return SM.sink_attention(
        q.to(dtype).to(device), cache, H, G, dk, vd, ints(table, device), bs, ints(cu, device),
        ints(seq, device), ints(pos, device), scale, softcap,
        None if sink is None else sink.to(device), None if talk is None else talk.to(device),
        dtype, tiles=ints(tiles, device).view(-1, 3), max_tile=mt).float().cpu()


@pytest.mark.parametrize("length,picks", [(30, [0, 1, 15, 16, 29]), (300, [0, 3, 127, 128, 255, 299])])
def test_attention_picks_one_key(dev, length, picks):
    """One key is made to stand out by scale: wherever it lies (the first
    tokens, a page's last and first row, far back), a prompt row and a
    decoded row must return exactly its value."""
    device, dtype = dev
    H, G, dk, vd, bs = 2, 2, 4, 3, 16
    g = torch.Generator().manual_seed(2)
    nb = (length + bs - 1) // bs
    table = torch.randperm(nb + 3, generator=g)[:nb].tolist()
    for pick in picks:
        k = 0.01 * torch.randn(length, G, dk, generator=g)
        v = torch.randn(length, G, vd, generator=g)
        k[pick] = torch.tensor([[3.0, 0, 0, 0], [0, 3.0, 0, 0]])
        cache = torch.zeros((nb + 3) * bs, G * (dk + vd), dtype=dtype, device=device)
        for j in range(length):
            cache[table[j // bs] * bs + j % bs] = torch.cat([k[j].reshape(-1), v[j].reshape(-1)]).to(dtype)
        q = torch.zeros(3, H, dk)
        q[:, 0, 0] = 10.0
        q[:, 1, 1] = 10.0
        # the last three positions as a prompt portion, then the last alone
        for pos in ([length - 3, length - 2, length - 1], [length - 1]):
            pos = [p for p in pos if p >= pick]
            out = _attend(dev, H, G, dk, vd, bs, [table], pos, cache, q[:len(pos)])
            want = v[pick].to(dtype).float().reshape(-1)
            for i in range(len(pos)):
                assert (out[i] - want).abs().max() < 2e-2, (pick, pos[i])


def test_attention_sink_cap_and_head_mixing(dev):
    device, dtype = dev
    H, G, dk, vd, bs = 4, 2, 4, 3, 4
    g = torch.Generator().manual_seed(3)
    n = 11
    k = torch.randn(n, G, dk, generator=g)
    v = torch.randn(n, G, vd, generator=g)
    table = [2, 0, 1]
    cache = torch.zeros(3 * bs, G * (dk + vd), dtype=dtype, device=device)
    for j in range(n):
        cache[table[j // bs] * bs + j % bs] = torch.cat([k[j].reshape(-1), v[j].reshape(-1)]).to(dtype)
    q = torch.randn(n, H, dk, generator=g)
    pos = list(range(n))
    t = 1e-5 if dtype == torch.float32 else 3e-2
    kk, vv = k.to(dtype).double(), v.to(dtype).double()
    qq = q.to(dtype).double()

    def plain(scale, cap, sink, talk):
        out = torch.zeros(n, H, vd, dtype=torch.float64)
        for i in range(n):
            w = torch.zeros(H, i + 1, dtype=torch.float64)
            for h in range(H):
                s = (kk[:i + 1, h // 2] @ qq[i, h]) * scale
                if cap:
                    s = cap * torch.tanh(s / cap)
                e = torch.exp(s)
                w[h] = e / (e.sum() + (torch.exp(sink[h].double()) if sink is not None else 0.0))
            if talk is not None:
                w = talk.double() @ w
            for h in range(H):
                out[i, h] = w[h] @ vv[:i + 1, h // 2]
        return out.reshape(n, -1)

    sink = torch.tensor([0.5, -1.0, 2.0, 0.0])
    talk = torch.eye(H) + 0.4 * torch.randn(H, H, generator=g)
    for scale, cap, sk, tk in [(0.5, 0.0, None, None), (0.5, 0.0, sink, None), (2.0, 1.5, None, None),
                               (0.5, 0.0, None, talk), (1.3, 2.0, sink, talk)]:
        got = _attend(dev, H, G, dk, vd, bs, [table], pos, cache, q, scale, cap, sk, tk)
        assert rel_err(got, plain(scale, cap, sk, tk)) < t, (scale, cap, sk is not None, tk is not None)
    # a dominant sink takes nearly all the weight; a cap levels two large scores
    big = _attend(dev, H, G, dk, vd, bs, [table], pos, cache, q, 0.5, 0.0, torch.full((H,), 30.0), None)
    assert big.abs().max() < 1e-6


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_conv_silu_portions(dev, taps):
    device, dtype = dev
    C, n = 7, 13
    g = torch.Generator().manual_seed(4)
    x = torch.randn(n, C + 2, generator=g).to(dtype)
    w = torch.randn(C, taps, generator=g)
    want = torch.stack(O.short_conv_silu([x[t, :C].double() for t in range(n)], w.double()))
    tails = torch.zeros(3, taps - 1, C, device=device)
    tails[1] = 5.0                                            # another sequence's slot
    got, at = [], 0
    for cnt in (1, 2, 5, 1, 4):
        xs = x[at:at + cnt].to(device)[:, :C]                 # a column slice of wider rows
        got.append(SM.tap_conv_silu(xs, w.to(device), tails, ints([0, cnt], device),
                                    ints([0] * cnt, device), ints([2], device), dtype))
        at += cnt
    assert rel_err(torch.cat(got), want) < (1e-6 if dtype == torch.float32 else 8e-3)
    assert bool((tails[1] == 5.0).all())


@pytest.mark.parametrize("H,G,dk,vd", [(4, 2, 8, 6), (2, 1, 40, 5), (3, 3, 5, 70), (2, 2, 72, 9)])
def test_delta_rule_against_oracle(dev, H, G, dk, vd):
    """The recurrence alone: identity projections turn the oracle's mixer
    into the op's inputs. Portions and a second row share the steps."""
    device, dtype = dev
    n, eps = 19, 1e-5
    g = torch.Generator().manual_seed(5)
    C = 2 * G * dk + H * vd
    D = C + H * vd + 2 * H                                    # [q k v | gate | b a]
    hs = torch.randn(n, D, generator=g).to(dtype).float()
    eye = torch.eye(D, dtype=torch.float64)
    W = {"q": eye[:G * dk], "k": eye[G * dk:2 * G * dk], "v": eye[2 * G * dk:C],
         "g": eye[C:C + H * vd], "b": eye[C + H * vd:C + H * vd + H], "a": eye[C + H * vd + H:],
         "A_log": 0.5 * torch.randn(H, generator=g).double(),
         "dt_bias": 0.5 * torch.randn(H, generator=g).double(),
         "norm": 1.0 + 0.1 * torch.randn(vd, generator=g).double(),
         "o": torch.eye(H * vd, dtype=torch.float64)}
    for nm, rows in (("q", G * dk), ("k", G * dk), ("v", H * vd)):
        W[nm + ".conv"] = torch.cat([torch.zeros(rows, 1), torch.ones(rows, 1)], 1).double()
    mc = {"heads": H, "kv_heads": G, "dim": dk, "vdim": vd}
    # the oracle applies conv + SiLU; feed the op the same activations
    want = torch.stack(O.delta_mixer([h.double() for h in hs], W, "", mc, eps))
    act = (hs[:, :C].double() * torch.sigmoid(hs[:, :C].double())).to(dtype)
    state = torch.zeros(3, H * dk * vd, device=device)
    other = torch.randn(4, C, generator=g).to(dtype)
    got, at = [], 0
    for cnt in (1, 2, 9, 1, 6):
        sl = slice(at, at + cnt)
        qkv = torch.cat([act[sl], other[:2]]).to(device)
        gate = torch.cat([hs[sl, C:C + H * vd], torch.zeros(2, H * vd)]).to(dtype).to(device)
        ab = torch.cat([hs[sl, C + H * vd:], torch.zeros(2, 2 * H)]).to(device)
        out = SM.gated_delta_rule(qkv, gate, ab, W["A_log"].float().to(device),
                                  W["dt_bias"].float().to(device), W["norm"].float().to(device), eps,
                                  state, ints([0, cnt, cnt + 2], device), ints([1, 2], device),
                                  H, G, dk, vd, dtype)
        got.append(out[:cnt])
        at += cnt
    assert rel_err(torch.cat(got), want) < (2e-5 if dtype == torch.float32 else 2e-2)
    assert float(state[0].abs().max()) == 0.0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,H,G,dk,vd", [(32, 32, 8, 32, 64), (16, 16, 4, 72, 40)])
def test_delta_rule_many_rows_layout(dtype, B, H, G, dk, vd):
    """With many rows and heads and several tokens per row the scan keeps
    32 state rows per lane instead of 8; the torch form of the op (itself
    held to the oracle on the CPU) must agree, two steps in a row so that
    the stored state is read back (the second by the 8-row form)."""
    from distrl_llm_amd.ops import seqmix_reference as R
    g = torch.Generator().manual_seed(11)
    C = 2 * G * dk + H * vd
    a_log, dtb = 0.5 * torch.randn(H, generator=g), 0.5 * torch.randn(H, generator=g)
    nw = 1.0 + 0.1 * torch.randn(vd, generator=g)
    st_cpu = torch.zeros(B + 1, H * dk * vd)
    st_gpu = st_cpu.clone().cuda()
    slots = torch.randperm(B + 1, generator=g)[:B].to(torch.int32)
    for step in range(2):
        lens = [(9 if step == 0 else 1) + (i % 3) for i in range(B)]
        T, cu = sum(lens), [0]
        for n in lens:
            cu.append(cu[-1] + n)
        qkv = torch.randn(T, C, generator=g).to(dtype)
        gate = torch.randn(T, H * vd, generator=g).to(dtype)
        ab = torch.randn(T, 2 * H, generator=g)
        want = R.gated_delta_rule(qkv.float(), gate.float(), ab, a_log, dtb, nw, 1e-5, st_cpu,
                                  torch.tensor(cu), slots, H, G, dk, vd, torch.float32)
        got = SM.gated_delta_rule(qkv.cuda(), gate.cuda(), ab.cuda(), a_log.cuda(), dtb.cuda(),
                                  nw.cuda(), 1e-5, st_gpu, ints(cu, "cuda"), slots.cuda(),
                                  H, G, dk, vd, dtype)
        assert rel_err(got, want) < (2e-5 if dtype == torch.float32 else 1e-2), step
    assert rel_err(st_gpu, st_cpu) < 2e-5


def test_capped_glu_and_router(dev):
    device, dtype = dev
    g = torch.Generator().manual_seed(6)
    T, D, ff = 9, 12, 7
    gu = (3.0 * torch.randn(T, 2 * ff, generator=g)).to(dtype)
    got = SM.capped_glu(gu.to(device), 1.25)
    a, b = gu[:, :ff].double().clamp(max=1.25), gu[:, ff:].double().clamp(-1.25, 1.25)
    assert rel_err(got, a * torch.sigmoid(1.702 * a) * (b + 1)) < (1e-6 if dtype == torch.float32 else 8e-3)
    # the correction decides the choice, not the weight
    h = torch.randn(T, D, generator=g).to(dtype)
    rw = torch.randn(6, D, generator=g)
    corr = torch.tensor([0.0, 0.0, 5.0, 0.0, 0.0, -5.0])
    idx, wts = SM.moe_route_all(h.to(device), rw.to(device), corr.to(device), 3, 1.5)
    s = torch.softmax(h.double() @ rw.double().T, -1)
    for t in range(T):
        want = torch.topk(s[t] + corr.double(), 3).indices.tolist()
        assert idx[t].tolist() == want and want[0] == 2 and 5 not in want
        assert rel_err(wts[t], 1.5 * s[t][want]) < 1e-5


@pytest.mark.parametrize("experts,identity,top,shared", [(5, 1, 2, True), (3, 0, 1, False), (2, 2, 4, True),
                                                        (4, 2, 3, False)])
def test_moe_layer(dev, experts, identity, top, shared):
    """One layer whose mixer is small beside its feed-forward: identity
    experts, top == experts + identity, no shared expert, top 1."""
    cfg = O.make_cfg([O.delta_layer(heads=1, kv_heads=1, dim=4, vdim=4, conv=2,
                                    mlp=O.mlp_cfg("moe", experts=experts, identity=identity, top=top,
                                                  shared=shared, ff=9))], width=12, vocab=23)
    W, eng = build(cfg, dev)
    t = toks(70, 23, seed=7)
    want, _ = O.forward(cfg, W, t)
    assert rel_err(run_portions(eng, t, [64, 1, 1, 4]), want) < tol(dev[1])


# ------------------------------------------------------------ whole model

def test_whole_prompt_and_layers(dev):
    cfg = mixed_cfg()
    W, eng = build(cfg, dev)
    t = toks(21, cfg["vocab"], seed=3)
    want, stream = O.forward(cfg, W, t)
    cap = []
    got = run_portions(eng, t, [21], capture=cap)
    assert len(cap) == len(cfg["layers"])
    for i, x in enumerate(cap):
        assert rel_err(x, stream[i]) < tol(dev[1]), i
    assert rel_err(got, want) < tol(dev[1])


@pytest.mark.parametrize("cuts", [[21], [1] * 21, [2] * 10 + [1], [3, 2, 7, 1, 1, 5, 2],
                                  [16, 1, 1, 1, 1, 1], [4, 4, 4, 4, 5]])
def test_portions_equal_whole(dev, cuts):
    cfg = mixed_cfg()
    W, eng = build(cfg, dev)
    t = toks(21, cfg["vocab"], seed=4)
    want, _ = O.forward(cfg, W, t)
    assert rel_err(run_portions(eng, t, cuts), want) < tol(dev[1])


def test_portions_are_exact_in_fp32(dev):
    """How a prompt is cut must not change the state or the logits beyond
    rounding: the recurrence walks tokens in order either way."""
    if dev[1] != torch.float32:
        pytest.skip("compared at fp32 accuracy")
    cfg = mixed_cfg()
    W, eng = build(cfg, dev)
    t = toks(40, cfg["vocab"], seed=5)
    a = run_portions(eng, t, [40])
    b = run_portions(eng, t, [7, 2, 2, 17, 1, 1, 10])
    assert rel_err(a, b) < 2e-6


def test_mixed_batch_equals_alone_with_reuse(dev):
    cfg = mixed_cfg()
    W, eng = build(cfg, dev, blocks=14, block_size=4, slots=3)
    reqs = {i: toks(n, cfg["vocab"], seed=10 + i) for i, n in enumerate([19, 7, 1, 12, 9, 16])}
    want = {i: O.forward(cfg, W, t)[0] for i, t in reqs.items()}
    plan = [
        [(0, 5), (1, 2), (2, 1)],
        [(0, 1), (1, 5), (3, 3)],
        [(0, 6), (3, 1), (4, 2)],
        [(3, 8), (4, 1)],
        [(0, 7), (4, 6), (5, 2)],
        [(5, 13)], [(5, 1)],
    ]
    live, at, got = {}, {i: 0 for i in reqs}, {i: [] for i in reqs}
    for rows in plan:
        work, wants = [], []
        for i, n in rows:
            if i not in live:
                live[i] = eng.open_sequence()
            work.append((live[i], reqs[i][at[i]:at[i] + n]))
            wants.append(list(range(n)))
        out = eng.step(work, wants)
        o = 0
        for i, n in rows:
            got[i].append(out[o:o + n])
            o += n
            at[i] += n
            if at[i] == len(reqs[i]):
                eng.close_sequence(live.pop(i))
    assert not live
    for i in reqs:
        assert rel_err(torch.cat(got[i]), want[i]) < tol(dev[1]), i
        # what else is in the batch changes nothing beyond rounding
        alone = run_portions(eng, reqs[i], [len(reqs[i])])
        assert rel_err(torch.cat(got[i]), alone) < (1e-5 if dev[1] == torch.float32 else 3e-2), i
    assert eng.pool.allocator.num_free == 14 and eng.slots.num_free == 3


def test_long_decode_far_key_and_old_state(dev):
    """Decoding runs over many pages. The weights make one early token
    matter at the end through the attention (a far key) and, separately,
    through the delta rule's state."""
    cfg = O.make_cfg([O.delta_layer(heads=2, kv_heads=1, dim=8, vdim=8, conv=2, mlp=None),
                      O.attn_layer(heads=2, kv_heads=1, dim=8, vdim=6, softcap=0.0, mlp="dense")],
                     width=12, vocab=17)
    W = O.random_weights(cfg, 0)
    W["l0.mix.A_log"] = torch.full((2,), -6.0)         # slow decay: the state remembers
    W, eng = build(cfg, dev, blocks=60, block_size=4, W=W)
    t = toks(150, 17, seed=9)
    want, _ = O.forward(cfg, W, t)
    got = run_portions(eng, t, [10] + [1] * 140)
    assert rel_err(got, want) < tol(dev[1])
    t2 = list(t)
    t2[3] = (t2[3] + 1) % 17
    assert rel_err(O.forward(cfg, W, t2)[0][-1], want[-1]) > 1e-5
    only_delta = O.make_cfg(cfg["layers"][:1], width=12, vocab=17)
    Wd = {k: v for k, v in W.items() if not k.startswith("l1.")}
    assert rel_err(O.forward(only_delta, Wd, t2)[0][-1], O.forward(only_delta, Wd, t)[0][-1]) > 1e-7


def test_long_prompt_beside_short_rows(dev):
    cfg = O.make_cfg([O.attn_layer(heads=4, kv_heads=2, dim=8, vdim=6, mlp=None),
                      O.delta_layer(heads=2, kv_heads=2, dim=8, vdim=6, conv=3, mlp="dense"),
                      O.attn_layer(heads=4, kv_heads=2, dim=8, vdim=6, rot_dims=4, mlp=None)],
                     width=12, vocab=13)
    W, eng = build(cfg, dev, blocks=80, block_size=4)
    a, b = toks(150, 13, seed=70), toks(5, 13, seed=71)
    qa, qb = eng.open_sequence(), eng.open_sequence()
    out = eng.step([(qa, a[:139]), (qb, b)], [list(range(139)), list(range(5))])
    out2 = eng.step([(qa, a[139:])], [list(range(11))])
    eng.close_sequence(qa)
    eng.close_sequence(qb)
    assert rel_err(torch.cat([out[:139], out2]), O.forward(cfg, W, a)[0]) < tol(dev[1])
    assert rel_err(out[139:], O.forward(cfg, W, b)[0]) < tol(dev[1])


def test_portions_cut_at_kernel_chunk_edges(dev):
    """The kernels work in chunks of their own (16-token scan chunks, 16-row
    and 64-query tiles, 64-key blocks, 16-token pages here): portions end
    just before, at and just after those edges, and single tokens are
    decoded across them."""
    cfg = O.make_cfg([O.attn_layer(heads=4, kv_heads=2, dim=8, vdim=8, softcap=6.0, mlp=None),
                      O.delta_layer(heads=2, kv_heads=1, dim=8, vdim=8, conv=4, mlp="dense")],
                     width=12, vocab=19)
    W, eng = build(cfg, dev, blocks=16, block_size=16)
    t = toks(196, 19, seed=77)
    want, _ = O.forward(cfg, W, t)
    cuts = [15, 1, 1, 46, 1, 1, 63, 1, 1, 2, 64]
    assert rel_err(run_portions(eng, t, cuts), want) < tol(dev[1])


def test_dirty_slot_and_pages_do_not_leak(dev):
    cfg = mixed_cfg()
    W, eng = build(cfg, dev, blocks=6, block_size=4, slots=1)
    a, b = toks(22, cfg["vocab"], seed=20), toks(13, cfg["vocab"], seed=21)
    run_portions(eng, a, [22])
    assert rel_err(run_portions(eng, b, [6, 7]), O.forward(cfg, W, b)[0]) < tol(dev[1])


def test_fork_shares_pages_and_copies_state(dev):
    cfg = mixed_cfg()
    W, eng = build(cfg, dev, blocks=20, block_size=4)
    t = toks(18, cfg["vocab"], seed=30)
    q = eng.open_sequence()
    eng.step([(q, t[:10])], [[]])
    c = eng.fork_sequence(q)
    tail2 = [(x + 3) % cfg["vocab"] for x in t[10:]]
    out = eng.step([(q, t[10:]), (c, tail2)], [list(range(8)), list(range(8))])
    assert rel_err(out[:8], O.forward(cfg, W, t)[0][10:]) < tol(dev[1])
    assert rel_err(out[8:], O.forward(cfg, W, t[:10] + tail2)[0][10:]) < tol(dev[1])
    eng.close_sequence(q)
    eng.close_sequence(c)
    assert eng.pool.allocator.num_free == 20


def oracle_greedy(cfg, W, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(cfg, W, seq)[0][-1].argmax()))
    return seq[len(prompt):]


def test_generate_greedy_through_scheduler(dev):
    if dev[1] == torch.bfloat16:
        pytest.skip("greedy token equality is checked in fp32")
    cfg = mixed_cfg()
    W, eng = build(cfg, dev, blocks=40, block_size=4, slots=4)
    prompts = [toks(n, cfg["vocab"], seed=40 + n) for n in (9, 3, 14, 1, 6)]
    want = [oracle_greedy(cfg, W, p, 6) for p in prompts]
    sp = SamplingParams(max_tokens=6, temperature=0.0, n=1)
    got = eng.generate(prompts, sp, prefill_token_budget=5)
    assert [g[0] for g in got] == want
    sp2 = SamplingParams(max_tokens=4, temperature=0.0, n=2)
    got2 = eng.generate(prompts[:2], sp2)
    for g, w in zip(got2, want):
        assert g[0] == w[:4] and g[1] == w[:4]
    assert eng.pool.allocator.num_free == 40 and eng.slots.num_free == 4


@pytest.mark.gpu
def test_captured_decode_equals_eager():
    cfg = mixed_cfg()
    dev = ("cuda", torch.float32)
    W, eng = build(cfg, dev, blocks=40, block_size=4, slots=4)
    eager = HybridEngine(eng.model, EngineConfig(max_seq_length=4096, kv_block_size=4, num_kv_blocks=40,
                                                 num_state_slots=4, max_num_seqs=4, enforce_eager=True),
                         device=torch.device("cuda"))
    prompts = [toks(n, cfg["vocab"], seed=60 + n) for n in (5, 11, 2)]
    outs = []
    for e in (eng, eager):
        qs = [e.open_sequence() for _ in prompts]
        e.step([(q, p) for q, p in zip(qs, prompts)])
        got = []
        for k in range(12):
            got.append(e.step([(q, [(7 * k + i) % cfg["vocab"]]) for i, q in enumerate(qs)]))
            if k == 5:
                e.step([(qs[0], [1, 2, 3])])
        for q in qs:
            e.close_sequence(q)
        outs.append(torch.stack(got))
    assert eng._decode_graphs and not eager._decode_graphs
    assert rel_err(outs[0], outs[1]) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk,vd,lens,talk", [(4, 2, 64, 48, [300, 1, 37, 2], True),
                                                 (6, 3, 128, 128, [70, 16, 17], True),
                                                 (4, 4, 32, 64, [129, 5], False),
                                                 (2, 1, 96, 40, [65, 33], True),
                                                 (8, 2, 128, 64, [1, 1, 1, 1], True),
                                                 (4, 4, 32, 64, [1, 1, 1], False),
                                                 (48, 8, 64, 32, [1, 1], True),
                                                 (6, 3, 40, 24, [1, 1, 1, 1], True),
                                                 (4, 4, 64, 160, [70, 3], True),
                                                 (4, 4, 64, 160, [1, 1, 1], True)])
def test_tiled_attention_kernel_against_plain_op(H, G, dk, vd, lens, talk):
    """bf16 prompt portions take the tiled MFMA kernel, steps of single
    tokens its heads-of-one-token form with split key ranges; the fp32
    reference op on the same cache rows must agree. Rows start at uneven
    positions inside their sequences and pages are scattered."""
    device, bs = torch.device("cuda"), 16
    g = torch.Generator().manual_seed(8)
    starts = [5, 40, 0, 330][:len(lens)]
    nb = [(s + n + bs - 1) // bs for s, n in zip(starts, lens)]
    perm = torch.randperm(sum(nb) + 2, generator=g).tolist()
    tables, at = [], 0
    for n in nb:
        tables.append(perm[at:at + n] + [0] * (max(nb) - n))
        at += n
    cache = torch.randn((sum(nb) + 2) * bs, G * (dk + vd), generator=g).to(torch.bfloat16).to(device)
    T = sum(lens)
    q = torch.randn(T, H, dk, generator=g).to(torch.bfloat16).to(device)
    pos, seq, cu = [], [], [0]
    for b, (s, n) in enumerate(zip(starts, lens)):
        pos += list(range(s, s + n))
        seq += [b] * n
        cu.append(cu[-1] + n)
    sink = torch.randn(H, generator=g).to(device)
    tk = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)).to(device) if talk else None
    tiles, mt = SM.query_tiles(lens, SM.WIDE_QUERY_TILE)
    args = (H, G, dk, vd, ints(tables, device), bs, ints(cu, device), ints(seq, device),
            ints(pos, device), dk ** -0.5, 4.0, sink, tk)
    got = SM.sink_attention(q, cache, *args, torch.bfloat16, tiles=ints(tiles, device).view(-1, 3),
                            max_tile=mt)
    from distrl_llm_amd.ops import seqmix_reference as R
    want = R.sink_attention(q.cpu().float(), cache.cpu().float(), H, G, dk, vd,
                            torch.tensor(tables), bs, torch.tensor(cu), torch.tensor(pos),
                            dk ** -0.5, 4.0, sink.cpu(), None if tk is None else tk.cpu(), torch.float32)
    assert rel_err(got, want) < 1e-2


def test_checkpoint_registry_and_trace_replay(tmp_path):
    from distrl_llm_amd.models.registry import load_model_and_engine
    cfg = mixed_cfg()
    W = O.random_weights(cfg, 3)
    model = HybridLM(nedasun_spec_from_config(cfg), dtype=torch.float32)
    model.load_tensors(W)
    ck = str(tmp_path / "ck")
    save_nedasun_checkpoint(model, ck)
    saved = json.load(open(os.path.join(ck, "config.json")))
    assert nedasun_spec_from_config(saved).layers == nedasun_spec_from_config(cfg).layers
    from safetensors.torch import load_file
    back = load_file(os.path.join(ck, "model.safetensors"))
    assert set(back) == set(W) and back["l2.mix.vmix"].shape == ()
    # the blend factor of layers that never read it may be left out; a tensor
    # the design does not name is ignored; anything else missing is an error
    from safetensors.torch import save_file
    trimmed = {k: v for k, v in back.items() if k not in ("l0.mix.vmix", "l2.mix.vmix")}
    trimmed["l0.mix.other"] = torch.zeros(3)
    save_file(trimmed, os.path.join(ck, "model.safetensors"))
    m2, eng = load_model_and_engine(ck, EngineConfig(num_kv_blocks=8, num_state_slots=2),
                                    dtype=torch.float32, device=torch.device("cpu"))
    assert isinstance(eng, HybridEngine) and m2.spec.block == "sandwich"
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    save_file({k: v for k, v in back.items() if k != "l4.mix.vmix"},
              os.path.join(bad, "model.safetensors"))
    json.dump(saved, open(os.path.join(bad, "config.json"), "w"))
    with pytest.raises(ValueError):
        load_model_and_engine(bad, EngineConfig(num_kv_blocks=8, num_state_slots=2),
                              dtype=torch.float32, device=torch.device("cpu"))
    a, b = toks(9, cfg["vocab"], seed=50), toks(5, cfg["vocab"], seed=51)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:4], "want": [3]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": a[4:8], "want": []},
                                     {"id": "y", "tokens": b, "want": [0, 4]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": a[8:], "want": [0]}], "end": ["x"]}]
    out = str(tmp_path / "out")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, HIP_VISIBLE_DEVICES="", CUDA_VISIBLE_DEVICES="")
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", ck,
                        "--dtype", "float32", "--out", out, "--max-tokens", "32", "--block-size", "4"],
                       input="".join(json.dumps(s) + "\n" for s in steps), text=True,
                       capture_output=True, env=env, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    la, lb = O.forward(cfg, W, a)[0], O.forward(cfg, W, b)[0]
    rd = lambda n: torch.from_numpy(np.fromfile(os.path.join(out, f"{n}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]).copy())
    assert rel_err(rd(0), la[3:4]) < 2e-4
    assert rel_err(rd(1), lb[[0, 4]]) < 2e-4
    assert rel_err(rd(2), la[8:9]) < 2e-4


def test_served_through_the_batcher():
    """The server's app, batcher and sampler drive the design's engine like
    any other: greedy completions repeat, sampled ones fan out, logprob
    rescoring uses the engine's own scoring pass."""
    from fastapi.testclient import TestClient

    from distrl_llm_amd.serve import create_app
    from distrl_llm_amd.utils.tokenizer import ByteTokenizer
    cfg = O.make_cfg([O.attn_layer(heads=4, kv_heads=2, dim=8, vdim=6, mlp="dense"),
                      O.delta_layer(heads=2, kv_heads=1, dim=8, vdim=6, conv=3, mlp="moe")],
                     width=16, vocab=600)
    _, eng = build(cfg, ("cpu", torch.float32), blocks=128, block_size=8, slots=8)
    client = TestClient(create_app(eng, ByteTokenizer(vocab_size=600), "tiny-nedasun"))
    body = {"prompt": "2+2=", "max_tokens": 5, "temperature": 0.0}
    a = client.post("/v1/completions", json=body).json()
    b = client.post("/v1/completions", json=body).json()
    assert a["choices"][0]["text"] == b["choices"][0]["text"]
    assert a["usage"]["completion_tokens"] <= 5
    r = client.post("/v1/completions", json={"prompt": ["abcd", "wxyz"], "max_tokens": 3,
                                             "temperature": 1.0, "top_p": 0.9, "n": 2}).json()
    assert len(r["choices"]) == 4
    lp = client.post("/v1/completions", json={"prompt": "ab", "max_tokens": 3, "temperature": 0.0,
                                              "logprobs": 1})
    assert lp.status_code == 200
    assert eng.pool.allocator.num_free == 128 and eng.slots.num_free == 8


def test_config_errors():
    cfg = mixed_cfg()
    for path, value in [((0, "type"), "other"), ((2, "mixer", "kv_heads"), 4),
                        ((2, "mixer", "rot", "dims"), 7), ((1, "mlp", "kind"), "sparse"),
                        ((6, "mixer", "v_mix"), True)]:      # 1 x 14 values cannot blend with 2 x 7
        bad = json.loads(json.dumps(cfg))
        node = bad["layers"][path[0]]
        for k in path[1:-1]:
            node = node[k]
        node[path[-1]] = value
        with pytest.raises(ValueError):
            nedasun_spec_from_config(bad)
