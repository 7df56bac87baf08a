"""Vigonex (residual streams with gated writes, token shift, differential
attention with a query temperature, the generalized delta rule, dense gated
or routed clamped experts with a gated shared expert) in the engine against
the plain oracle in vigonex_oracle.py: every mechanism alone, prompt vs
token-by-token decoding, prompt portions down to two tokens, unequal batches,
reuse of freed cache blocks and state slots, keys far back and at page
borders (planted so that one score stands out), first tokens, long decoding,
other sizes, and greedy generation through the engine's own scheduler. CPU
runs use the torch reference ops; the same cases run on the GPU kernels under
the gpu marker, where the kernels are also compared one by one with the
reference ops.
"""
import json
import math
import os

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import vigonex_oracle as oracle
from kubeai_amd.engine import EngineConfig, LLMEngine, SamplingParams
from kubeai_amd.ops import seq as sops

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
GPU = [pytest.param("cuda", marks=pytest.mark.gpu)]

DENSE = {"kind": "dense", "ff": 40}


def moe(experts=5, top=2, ff=12, limit=1.0, scale=1.3, shared=(10, 0.8)):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
         "router": {"experts": experts, "top": top, "scale": scale}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


MOE = moe()


def att(heads=4, kv=2, dim=6, vdim=10, diff=0.2, scale=0.4, softcap=5.0, temp=(0.5, 3),
        mlp=DENSE):
    mx = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "diff": diff,
          "scale": scale}
    if softcap:
        mx["softcap"] = softcap
    if temp:
        mx["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def delta(heads=2, dim=8, lowrank=5, mlp=MOE):
    return {"type": "general_delta", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "lowrank": lowrank}}


def config(layers, width=24, vocab=40, eps=1e-5, streams=3, emb=2.0, logit=0.7):
    return {"architecture": "Vigonex", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "streams": streams, "embedding": {"scale": emb},
            "logit_scale": logit, "layers": layers}


MIXED = config([att(), delta(), att(heads=3, kv=1, dim=4, vdim=4, temp=(0.3, 16), mlp=MOE),
                delta(heads=1, dim=16, lowrank=3, mlp=None)])


def model_dir(tmp_path, cfg, seed=0, W=None):
    d = str(tmp_path / ("m%d" % seed))
    os.makedirs(d, exist_ok=True)
    W = W if W is not None else oracle.random_weights(cfg, seed)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()},
              os.path.join(d, "model.safetensors"))
    return d, oracle.as_float64(W)


def engine(d, device, dtype="float32", blocks=64, seqs=4):
    return LLMEngine(EngineConfig(
        model=d, device=device, dtype=dtype, num_gpu_blocks=blocks,
        max_num_seqs=seqs, max_model_len=1 << 20, max_num_batched_tokens=1 << 20,
        enable_prefix_caching=False, enable_graphs=False))


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(7000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_err(got, want):
    got = got.double().cpu().numpy() if isinstance(got, torch.Tensor) else got
    return np.abs(got - want).max(-1) / want.std()


def check(got, want, dtype="float32", loose=0.2):
    err = rel_err(got, want).max()
    # bf16: the widths here are tiny, so roundings do not average out
    assert err < (3e-4 if dtype == "float32" else loose), f"relative error {err:.3g}"


def replay(eng, rid, toks, cuts):
    """Feed toks in portions of the given sizes (the last repeats), wanting
    every position; returns [T, vocab]."""
    rows, at, i = [], 0, 0
    while at < len(toks):
        n = min(cuts[min(i, len(cuts) - 1)], len(toks) - at)
        part = toks[at : at + n]
        at += n
        i += 1
        out = eng.step_fixed([(rid, part, list(range(n)))],
                             [rid] if at == len(toks) else [])
        rows.append(out[0])
    return torch.cat(rows)


def npy(t):
    return t.detach().double().cpu().numpy()


def meta_of(runs, positions, device, tables=None):
    return sops.SeqMeta.build(runs, torch.tensor(positions, dtype=torch.int32, device=device),
                              device, block_tables=tables)


# ---------------------------------------------------------------------------
# mechanisms as functions: the product's ops against the oracle's
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("width,copies", [(24, 3), (7, 1), (130, 2)])
def test_embedding_with_position_vectors(device, width, copies):
    from kubeai_amd.models.vigonex import sinusoid_frequencies

    g = torch.Generator().manual_seed(width)
    table = torch.randn(11, width, generator=g)
    ids = [3, 0, 10, 3, 7, 1]
    pos = [0, 1, 63, 64, 900, 250000]
    got = sops.embed_sinusoid(torch.tensor(ids, dtype=torch.int32, device=device),
                              table.to(device), 1.7,
                              torch.tensor(pos, dtype=torch.int32, device=device),
                              sinusoid_frequencies(width).to(device), copies)
    assert got.shape == (6, copies, width) and got.dtype == torch.float32
    want = npy(table)[ids] * 1.7 + oracle.position_vectors(250001, width)[pos]
    for s in range(copies):
        assert np.abs(npy(got[:, s]) - want).max() < 2e-6
    # position 0: sines vanish, cosines are one
    assert np.allclose(npy(got[0, 0]) - npy(table)[3] * 1.7,
                       np.arange(width) % 2, atol=1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S", [1, 2, 3, 5])
def test_stream_update_read_and_norm(device, S):
    g = torch.Generator().manual_seed(S)
    T, C = 6, 20
    X = torch.randn(T, S, C, generator=g)
    y = torch.randn(T, C, generator=g)
    gate = torch.randn(T, C + 4, generator=g)[:, 2 : C + 2]  # strided rows
    mix = torch.randn(S, S, generator=g)  # not symmetric: [from, to] matters
    wr, rd, w = torch.randn(S, generator=g), torch.randn(S, generator=g), torch.rand(C, generator=g)
    z = npy(y) * oracle.sigmoid(npy(gate))
    Xn = np.einsum("st,nsc->ntc", npy(mix), npy(X)) + npy(wr)[None, :, None] * z[:, None]
    want = oracle.unit_rms(np.einsum("s,nsc->nc", npy(rd), Xn), 1e-5) * npy(w)
    Xd = X.to(device).clone()
    got = sops.hyper_mix_rmsnorm(Xd, y.to(device), gate.to(device), mix.to(device),
                                 wr.to(device), rd.to(device), w.to(device), 1e-5,
                                 torch.float32)
    assert np.abs(npy(got) - want).max() < 1e-5
    assert np.abs(npy(Xd) - Xn).max() < 1e-5
    # without a pending branch the streams stay and are only read
    Xd = X.to(device).clone()
    got = sops.hyper_mix_rmsnorm(Xd, None, None, None, None, rd.to(device), w.to(device),
                                 1e-5, torch.float32)
    want = oracle.unit_rms(np.einsum("s,nsc->nc", npy(rd), npy(X)), 1e-5) * npy(w)
    assert np.abs(npy(got) - want).max() < 1e-5 and torch.equal(Xd.cpu(), X)
    # an fp32 branch without a gate
    Xd = X.to(device).clone()
    sops.hyper_mix_rmsnorm(Xd, y.to(device), None, mix.to(device), wr.to(device),
                           rd.to(device), w.to(device), 1e-5, torch.float32)
    Xn = np.einsum("st,nsc->ntc", npy(mix), npy(X)) + npy(wr)[None, :, None] * npy(y)[:, None]
    assert np.abs(npy(Xd) - Xn).max() < 1e-5


@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_carries_the_previous_token(device):
    g = torch.Generator().manual_seed(1)
    C = 12
    h = torch.randn(9, C, generator=g)
    mu = torch.rand(1, C, generator=g)
    want = oracle.token_shift(npy(h), npy(mu[0]))
    prev = torch.full((3, 1, C), 99.0, device=device)  # stale slot contents
    got = []
    for lo, hi in ((0, 4), (4, 5), (5, 7), (7, 9)):
        meta = meta_of([(hi - lo, 2)], list(range(lo, hi)), device)
        got.append(sops.token_shift_mix(h[lo:hi].to(device), mu.to(device), prev, meta)[0])
    assert np.abs(npy(torch.cat(got)) - want).max() < 1e-6


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("coef,every", [(0.5, 3), (0.25, 48), (1.0, 1), (0.0, 5)])
def test_query_temperature_and_cache_rows(device, coef, every):
    g = torch.Generator().manual_seed(every)
    H, G, Gv, D, Dv, bs = 4, 4, 2, 6, 10, 4
    pos = [0, 1, 2, 3, 5, 46, 47, 48, 94, 95, 96, 143]  # both sides of every step of the floor
    T = len(pos)
    q, k, v = (torch.randn(T, n, d, generator=g) for n, d in ((H, D), (G, D), (Gv, Dv)))
    kc, vc = torch.zeros(60, G, bs, D, device=device), torch.zeros(60, Gv, bs, Dv, device=device)
    slots = torch.tensor([p + 7 for p in pos], dtype=torch.int64)
    slots[4] = -1  # padding rows are not written
    qd = q.to(device).clone()
    sops.scale_q_and_cache(qd, k.to(device), v.to(device),
                           torch.tensor(pos, dtype=torch.int32, device=device), coef, every,
                           kc, vc, slots.to(device))
    temp = oracle.query_temperature(144, {"coef": coef, "every": every} if coef else None)
    assert np.abs(npy(qd) - npy(q) * temp[pos][:, None, None]).max() < 1e-5
    for i, p in enumerate(pos):
        s = p + 7
        if i == 4:
            assert float(kc[s // bs, :, s % bs].abs().max()) == 0.0
            continue
        assert torch.equal(kc[s // bs, :, s % bs].cpu(), k[i])
        assert torch.equal(vc[s // bs, :, s % bs].cpu(), v[i])


def _attend(device, q, k, v, scale, softcap, cuts, block=16, dtype=torch.float32, seed=0):
    """q [T, Hq, D], k [T, Gk, D], v [T, Gv, Dv] through the paged attention op
    in portions; the blocks of the one sequence lie scattered."""
    T, Hq, D = q.shape
    Gk, Gv, Dv = k.shape[1], v.shape[1], v.shape[2]
    nblk = (T + block - 1) // block
    perm = torch.randperm(nblk + 3, generator=torch.Generator().manual_seed(T + seed)).tolist()
    table = torch.tensor([perm[:nblk]], dtype=torch.int32, device=device)
    kc = torch.zeros(nblk + 3, Gk, block, D, device=device, dtype=dtype)
    vc = torch.zeros(nblk + 3, Gv, block, Dv, device=device, dtype=dtype)
    outs, at = [], 0
    for n in cuts:
        n = min(n, T - at)
        pos = torch.arange(at, at + n)
        slot = (table[0].cpu()[pos // block].long() * block + pos % block).to(device)
        qq = q[at : at + n].to(device, dtype).contiguous()
        sops.scale_q_and_cache(qq, k[at : at + n].to(device, dtype), v[at : at + n].to(device, dtype),
                               pos.to(device, torch.int32), 0.0, 1, kc, vc, slot)
        meta = meta_of([(n, 0)], pos.tolist(), device, table)
        out = torch.zeros(n, Hq, Dv, device=device, dtype=dtype)
        sops.masked_paged_attention(qq, kc, vc, meta, scale, out, softcap=softcap)
        outs.append(out)
        at += n
        if at >= T:
            break
    return torch.cat(outs)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 6, 10), (3, 3, 4, 4), (1, 1, 16, 16), (6, 1, 8, 2)])
def test_two_score_maps_over_shared_value_heads(device, H, G, D, Dv):
    """Key heads 2 g + m, value heads g, query heads in (group, map, head)
    order: every query head meets its own key head and its group's values."""
    g = torch.Generator().manual_seed(H * 10 + G)
    T, R = 37, H // G
    q = torch.randn(T, G, 2, R, D, generator=g)
    k = torch.randn(T, G, 2, D, generator=g)
    v = torch.randn(T, G, Dv, generator=g)
    got = _attend(device, q.view(T, 2 * H, D), k.view(T, 2 * G, D), v, 0.6, 4.0, [20, 1, 1, 15])
    got = got.view(T, G, 2, R, Dv)
    for gi in range(G):
        for m in range(2):
            for r in range(R):
                want = oracle.causal_softmax_attention(npy(q[:, gi, m, r]), npy(k[:, gi, m]),
                                                       npy(v[:, gi]), 0.6, 4.0)
                assert np.abs(npy(got[:, gi, m, r]) - want).max() < 1e-5, (gi, m, r)
    # the join: difference, per-head RMS norm, gain
    out = torch.zeros(T, H, Dv, device=device)
    sops.diff_combine(got, 0.7, 0.8, 1e-5, out)
    a = npy(got)
    want = oracle.unit_rms(a[:, :, 0] - 0.7 * a[:, :, 1], 1e-5).reshape(T, H, Dv) * 0.8
    assert np.abs(npy(out) - want).max() < 1e-5


FAR = [(99, 90), (47, 32), (47, 31), (48, 47), (700, 3), (1029, 0), (5, 0), (15, 15), (16, 16)]


def _planted(device, q_pos, key_pos, decode, dims=(2, 1, 8, 8), dtype=torch.float32, boost=30.0):
    """Random keys, but in map 1 of group 0 the key at key_pos and the query
    at q_pos are aligned and long: that map's output at q_pos is the value at
    key_pos; map 0 stays diffuse."""
    H, G, D, Dv = dims
    T, R = q_pos + 1, H // G
    g = torch.Generator().manual_seed(q_pos * 31 + key_pos)
    q = 0.3 * torch.randn(T, G, 2, R, D, generator=g)
    k = 0.3 * torch.randn(T, G, 2, D, generator=g)
    v = torch.randn(T, G, Dv, generator=g)
    k[key_pos, 0, 1] = 0.0
    k[key_pos, 0, 1, 0] = boost
    q[q_pos, 0, 1, :, 0] = boost / 10
    cuts = [q_pos, 1] if decode and q_pos else [T]
    got = _attend(device, q.view(T, 2 * H, D), k.view(T, 2 * G, D), v, 1.0, 0.0, cuts, dtype=dtype)
    got = got.view(T, G, 2, R, Dv)[q_pos, 0]
    want = np.stack([[oracle.causal_softmax_attention(npy(q[:, 0, m, r]), npy(k[:, 0, m]),
                                                      npy(v[:, 0]), 1.0, 0.0)[q_pos]
                      for r in range(R)] for m in range(2)])
    return npy(got.float()), want, npy(v[key_pos, 0])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("q_pos,key_pos", FAR)
def test_planted_key_far_back_and_at_page_borders(device, decode, q_pos, key_pos):
    got, want, value = _planted(device, q_pos, key_pos, decode)
    assert np.abs(want[1] - value).max() < 1e-6  # the planted key takes all the weight
    assert np.abs(want[0] - value).max() > 0.1 or q_pos == 0
    assert np.abs(got - want).max() < 1e-4


@pytest.mark.parametrize("device", GPU)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("dims", [(8, 2, 32, 64), (16, 1, 64, 128), (4, 4, 16, 16)])
@pytest.mark.parametrize("q_pos,key_pos", FAR)
def test_planted_key_matrix_core_kernels(device, decode, dims, q_pos, key_pos):
    got, want, value = _planted(device, q_pos, key_pos, decode, dims=dims, dtype=torch.bfloat16)
    assert np.abs(got[1] - value).max() < 0.05
    assert np.abs(got - want).max() < 0.05


def _delta_inputs(T, H, D, Dv, seed):
    g = torch.Generator().manual_seed(seed)
    r, k, wp, ap = (torch.randn(T, H, D, generator=g) for _ in range(4))
    v = torch.randn(T, H, Dv, generator=g)
    wb, ab = 1.5 * torch.randn(H * D, generator=g), torch.randn(H * D, generator=g)
    return r, k, v, wp, ap, wb, ab


def _delta_want(r, k, v, wp, ap, wb, ab, scale):
    T, H, D = k.shape
    w = np.exp(-scale * oracle.sigmoid(npy(wp) + npy(wb).reshape(H, D)))
    a = oracle.sigmoid(npy(ap) + npy(ab).reshape(H, D))
    return np.stack([oracle.general_delta_recurrence(npy(r[:, h]), npy(k[:, h]), npy(v[:, h]),
                                                     w[:, h], a[:, h]) for h in range(H)], 1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,Dv", [(2, 8, 8), (1, 16, 16), (3, 48, 48), (2, 10, 6), (1, 64, 64),
                                    (2, 24, 24)])
def test_delta_scan_function_and_carried_state(device, H, D, Dv):
    T = 45
    ins = _delta_inputs(T, H, D, Dv, D)
    scale = math.exp(-0.5)
    want = _delta_want(*ins, scale)
    r, k, v, wp, ap, wb, ab = (x.to(device) for x in ins)
    state = torch.full((3, H, D, Dv), 50.0, device=device)  # a stale slot
    got = []
    for lo, hi in ((0, 17), (17, 18), (18, 20), (20, 21), (21, 45)):
        meta = meta_of([(hi - lo, 1)], list(range(lo, hi)), device)
        got.append(sops.diag_rank1_scan(r[lo:hi], k[lo:hi], v[lo:hi], wp[lo:hi], ap[lo:hi],
                                        wb, ab, state, meta, scale))
    got = npy(torch.cat(got))
    assert np.abs(got - want).max() < 2e-4 * max(1.0, np.abs(want).max())
    # one call over the same tokens
    meta = meta_of([(T, 0)], list(range(T)), device)
    one = npy(sops.diag_rank1_scan(r, k, v, wp, ap, wb, ab, state, meta, scale))
    assert np.abs(one - want).max() < 2e-4 * max(1.0, np.abs(want).max())
    assert np.abs(npy(state[0]) - npy(state[1])).max() < 1e-3 * max(1.0, float(state[0].abs().max()))


@pytest.mark.parametrize("device", DEVICES)
def test_delta_scan_unequal_batch_and_long_run(device):
    H, D = 2, 16
    lens, slots = [300, 1, 7, 2], [2, 0, 3, -1]
    scale = math.exp(-0.5)
    parts = [_delta_inputs(n, H, D, D, 100 + i) for i, n in enumerate(lens)]
    wb, ab = parts[0][5], parts[0][6]
    cat = [torch.cat([p[j] for p in parts]).to(device) for j in range(5)]
    pos = [p for n in lens for p in range(n)]
    state = torch.zeros(4, H, D, D, device=device)
    meta = meta_of(list(zip(lens, slots)), pos, device)
    got = npy(sops.diag_rank1_scan(*cat, wb.to(device), ab.to(device), state, meta, scale))
    at = 0
    for p, n in zip(parts, lens):
        want = _delta_want(*p[:5], wb, ab, scale)
        assert np.abs(got[at : at + n] - want).max() < 3e-4 * max(1.0, np.abs(want).max())
        at += n


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_removes_what_a_key_held(device):
    """Unit keys along one axis, removal rate 1, no decay: a second write with
    the same key replaces the first value instead of adding to it; with
    removal rate 0 the values add up."""
    H, D = 1, 8
    k = torch.zeros(3, H, D)
    k[:, 0, 2] = 1.0
    r = k.clone()
    v = torch.tensor([[1.0] * D, [5.0] * D, [0.0] * D]).view(3, H, D)
    wp = torch.full((3, H, D), -40.0)  # sigmoid -> 0, decay factor 1
    zero = torch.zeros(H * D)
    for ap, want in ((40.0, [1.0, 5.0, 0.0]), (-40.0, [1.0, 6.0, 6.0])):
        state = torch.zeros(1, H, D, D, device=device)
        meta = meta_of([(3, 0)], [0, 1, 2], device)
        o = sops.diag_rank1_scan(r.to(device), k.to(device), v.to(device), wp.to(device),
                                 torch.full((3, H, D), ap).to(device), zero.to(device),
                                 zero.to(device), state, meta, 1.0)
        assert np.allclose(npy(o[:, 0, 0]), want, atol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_router_weights_scale_and_clamped_activation(device):
    z = torch.tensor([[0.1, 2.0, -1.0, 2.0, 0.5], [3.0, -3.0, 0.0, 1.0, 2.9]])
    dense, w, idx = sops.router_scores_topk(z.to(device), 2, None, 1.7)
    s = torch.softmax(z, -1)
    assert idx.cpu().tolist() == [[1, 3], [0, 4]]  # ties: the lower index first
    assert np.allclose(npy(w), npy(torch.gather(s, 1, idx.cpu().long()) * 1.7), atol=1e-6)
    assert np.allclose(npy(dense).sum(-1), npy(w).sum(-1), atol=1e-6)
    g = torch.Generator().manual_seed(5)
    gu = 3.0 * torch.randn(7, 2 * 3 * 8, generator=g)  # three experts of 8
    rw = torch.rand(7, 3, generator=g)
    got = sops.glu_weighted(gu.to(device), rw.to(device), 8, alpha=1.702, limit=1.8, up_shift=1.0)
    a = npy(gu).reshape(7, 3, 2, 8)
    gate, up = np.minimum(a[:, :, 0], 1.8), np.clip(a[:, :, 1], -1.8, 1.8)
    want = gate * oracle.sigmoid(1.702 * gate) * (up + 1.0) * npy(rw)[:, :, None]
    assert np.abs(npy(got) - want.reshape(7, 24)).max() < 1e-5
    # no weight, no clamp: plain silu(gate) * up; sigmoid of the weight column
    got = sops.glu_weighted(gu.to(device), None, 8)
    want = a[:, :, 0] * oracle.sigmoid(a[:, :, 0]) * a[:, :, 1]
    assert np.abs(npy(got) - want.reshape(7, 24)).max() < 1e-4
    wide = torch.zeros(7, 30, device=device)
    sops.glu_weighted(gu.to(device)[:, 16:32], rw.to(device)[:, 1:2], 8, w_sigmoid=True,
                      out=wide[:, 3:11])
    want = a[:, 1, 0] * oracle.sigmoid(a[:, 1, 0]) * a[:, 1, 1] * oracle.sigmoid(npy(rw)[:, 1:2])
    assert np.abs(npy(wide[:, 3:11]) - want).max() < 1e-4 and float(wide[:, 11:].abs().max()) == 0


# ---------------------------------------------------------------------------
# the engine against whole-sequence oracle runs
# ---------------------------------------------------------------------------
SINGLE = {
    "attention": config([att(mlp=None)]),
    "attention_dense": config([att()]),
    "attention_moe": config([att(mlp=MOE)]),
    "delta": config([delta(mlp=None)]),
    "delta_dense": config([delta(mlp=DENSE)]),
    "two_attention": config([att(mlp=None), att(heads=2, kv=2, mlp=None)]),
    "two_delta": config([delta(mlp=None), delta(heads=3, dim=4, mlp=None)]),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_whole_prompt(tmp_path, device, name):
    cfg = SINGLE[name]
    d, W = model_dir(tmp_path, cfg, seed=1)
    toks = tokens(29, cfg["vocab"], 1)
    got = replay(engine(d, device), "a", toks, [len(toks)])
    check(got, oracle.forward(cfg, W, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_streams_match_after_every_layer(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=2)
    toks = tokens(21, MIXED["vocab"], 2)
    eng = engine(d, device)
    eng.runner.model.capture_layers = []
    replay(eng, "a", toks, [len(toks)])
    want = []
    oracle.forward(MIXED, W, toks, want)
    got = eng.runner.model.capture_layers
    assert len(got) == len(want) == len(MIXED["layers"])
    for i, (a, b) in enumerate(zip(got, want)):
        a = npy(a)[: len(toks)]  # a step may be padded to a bucket
        assert np.abs(a - b).max() < 2e-4 * max(1.0, np.abs(b).max()), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2, 5], [7, 1, 1, 4, 1], [16, 1], [11, 13]])
def test_portions_and_token_by_token(tmp_path, device, cuts):
    d, W = model_dir(tmp_path, MIXED, seed=3)
    toks = tokens(38, MIXED["vocab"], 3)
    check(replay(engine(d, device), "a", toks, cuts), oracle.forward(MIXED, W, toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n", [1, 2, 3])
def test_first_tokens(tmp_path, device, n):
    d, W = model_dir(tmp_path, MIXED, seed=4)
    toks = tokens(n, MIXED["vocab"], 4)
    want = oracle.forward(MIXED, W, toks)
    check(replay(engine(d, device), "a", toks, [n]), want)
    check(replay(engine(d, device), "b", toks, [1]), want)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=5)
    toks = tokens(150, MIXED["vocab"], 5)
    check(replay(engine(d, device), "a", toks, [6, 1]), oracle.forward(MIXED, W, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_long_prompt_in_one_step_and_routed_path(tmp_path, device):
    """More than 256 tokens in a step take the per-expert gather path of the
    routed feed-forward; the same prompt in portions takes the dense one."""
    cfg = config([att(mlp=MOE), delta()], streams=2)
    d, W = model_dir(tmp_path, cfg, seed=6)
    toks = tokens(300, cfg["vocab"], 6)
    want = oracle.forward(cfg, W, toks)
    check(replay(engine(d, device), "a", toks, [300]), want)
    check(replay(engine(d, device), "b", toks, [270, 2, 1]), want)


OTHER = {
    # values that are equal or 1 in one place differ or are larger in another
    "one_stream": config([att(), delta()], streams=1),
    "five_streams": config([att(mlp=MOE), delta(mlp=DENSE)], streams=5),
    "every_head_its_own_key": config([att(heads=3, kv=3, dim=8, vdim=8)]),
    "one_head": config([att(heads=1, kv=1, dim=4, vdim=6), delta(heads=1, dim=4)]),
    "one_key_head": config([att(heads=6, kv=1, dim=2, vdim=12)]),
    "no_cap_no_temperature": config([att(softcap=0.0, temp=None)]),
    "temperature_every_token": config([att(temp=(1.0, 1))]),
    "no_difference_offset": config([att(diff=0.0)]),
    "top_one": config([att(mlp=moe(experts=3, top=1))]),
    "all_experts": config([att(mlp=moe(experts=3, top=3, scale=1.0))]),
    "one_expert": config([delta(mlp=moe(experts=1, top=1))]),
    "no_shared_expert": config([att(mlp=moe(shared=None))]),
    "wide_limits": config([delta(mlp=moe(limit=50.0, shared=(6, 50.0)))]),
    "sixteens": config([att(heads=4, kv=2, dim=16, vdim=32, mlp=moe(ff=16, shared=(32, 1.0))),
                        delta(heads=2, dim=16, lowrank=8, mlp={"kind": "dense", "ff": 64})],
                       width=64, vocab=80, streams=2, emb=1.0, logit=1.0),
    "odd_width": config([att(), delta()], width=23),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_sizes(tmp_path, device, name):
    cfg = OTHER[name]
    d, W = model_dir(tmp_path, cfg, seed=7)
    toks = tokens(26, cfg["vocab"], 7)
    check(replay(engine(d, device), "a", toks, [9, 2, 1]), oracle.forward(cfg, W, toks))


@pytest.mark.parametrize("device", GPU)
@pytest.mark.parametrize("name", ["sixteens", "odd_width"])
def test_bfloat16_serving_precision(tmp_path, device, name):
    cfg = OTHER[name]
    d, W = model_dir(tmp_path, cfg, seed=8)
    toks = tokens(70, cfg["vocab"], 8)
    want = oracle.forward(cfg, W, toks)
    a = replay(engine(d, device, "bfloat16"), "a", toks, [70])
    b = replay(engine(d, device, "bfloat16"), "b", toks, [33, 2, 1])
    check(a, want, "bfloat16")
    check(b, want, "bfloat16")


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_matches_each_alone(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=11)
    lens = {"a": 41, "b": 3, "c": 18, "d": 1}
    toks = {r: tokens(n, MIXED["vocab"], 10 + i) for i, (r, n) in enumerate(lens.items())}
    want = {r: oracle.forward(MIXED, W, t) for r, t in toks.items()}
    eng = engine(d, device)
    at = {r: 0 for r in toks}
    got = {r: [] for r in toks}
    plan = {"a": [5, 1, 1, 9, 2], "b": [1], "c": [2, 7, 1], "d": [1]}
    step = 0
    while any(at[r] < lens[r] for r in toks):
        entries, end = [], []
        for r in toks:
            if at[r] >= lens[r] or (r == "c" and step % 3 == 1):  # c sits some steps out
                continue
            n = min(plan[r][min(step, len(plan[r]) - 1)], lens[r] - at[r])
            entries.append((r, toks[r][at[r] : at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == lens[r]:
                end.append(r)
        for (r, _, _), rows in zip(entries, eng.step_fixed(entries, end)):
            got[r].append(rows)
        step += 1
    for r in toks:
        check(torch.cat(got[r]), want[r])
    assert eng.block_manager.num_free_blocks == eng.block_manager.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_freed_blocks_and_slots_are_reused(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=12)
    eng = engine(d, device, blocks=5, seqs=2)  # 80 tokens, two state slots
    for i in range(4):
        ta, tb = tokens(40 + i, MIXED["vocab"], 20 + i), tokens(17, MIXED["vocab"], 40 + i)
        ra, rb = "a%d" % i, "b%d" % i
        out = eng.step_fixed([(ra, ta[:30], list(range(30))), (rb, tb[:2], [0, 1])])
        ga, gb = [out[0]], [out[1]]
        out = eng.step_fixed([(rb, tb[2:], list(range(15))), (ra, ta[30:31], [0])], [rb])
        gb.append(out[0])
        ga.append(out[1])
        out = eng.step_fixed([(ra, ta[31:], list(range(len(ta) - 31)))], [ra])
        ga.append(out[0])
        check(torch.cat(ga), oracle.forward(MIXED, W, ta))
        check(torch.cat(gb), oracle.forward(MIXED, W, tb))
    with pytest.raises(Exception):
        eng.step_fixed([("x", tokens(81, MIXED["vocab"], 0), [])])


@pytest.mark.parametrize("device", DEVICES)
def test_far_token_reaches_logits(tmp_path, device):
    """Two prompts that differ in their first token only: through attention
    the last position still sees it; in a model of delta layers alone it is
    only the carried state that keeps it."""
    for name, cfg in (("att", config([att(mlp=None)], streams=2)),
                      ("delta", config([delta(mlp=None)], streams=2))):
        d, W = model_dir(tmp_path, cfg, seed=30 + len(name))
        base = tokens(420, cfg["vocab"], 30)
        other = [(base[0] + 1) % cfg["vocab"]] + base[1:]
        rows = {}
        for rid, toks in (("x", base), ("y", other)):
            eng = engine(d, device, blocks=40)
            got = replay(eng, rid, toks, [400, 17, 1])
            want = oracle.forward(cfg, W, toks)
            check(got[-4:], want[-4:])
            rows[rid] = want[-1]
        if name == "att":
            assert np.abs(rows["x"] - rows["y"]).max() > 1e-3 * rows["x"].std()


def test_unconsumed_and_missing_tensors_are_errors(tmp_path):
    cfg = SINGLE["attention_moe"]
    W = oracle.random_weights(cfg, 0)
    extra = dict(W, **{"l0.mix.extra": torch.zeros(3).bfloat16()})
    d, _ = model_dir(tmp_path, cfg, seed=40, W=extra)
    with pytest.raises(ValueError, match="not consumed"):
        engine(d, "cpu")
    less = {k: v for k, v in W.items() if k != "l0.mlp.shared.sg"}
    d, _ = model_dir(tmp_path, cfg, seed=41, W=less)
    with pytest.raises(ValueError, match="lacks"):
        engine(d, "cpu")
    with pytest.raises(ValueError):
        from kubeai_amd.models.config import vigonex_arch_config
        vigonex_arch_config(dict(cfg, streams=0))


def test_decay_bottleneck_size_comes_from_the_checkpoint(tmp_path):
    cfg = config([delta(lowrank=7, mlp=None)])
    W = oracle.random_weights(cfg, 3)
    del cfg["layers"][0]["mixer"]["lowrank"]  # the config does not say it
    d, W64 = model_dir(tmp_path, cfg, seed=42, W=W)
    toks = tokens(12, cfg["vocab"], 42)
    check(replay(engine(d, "cpu"), "a", toks, [5, 1]), oracle.forward(cfg, W64, toks))


# ---------------------------------------------------------------------------
# generation through the engine's own entry point and scheduler
# ---------------------------------------------------------------------------
def _generate(eng, prompts, max_tokens, arrive_every=0):
    pending = list(prompts.items())
    if not arrive_every:
        for rid, t in pending:
            eng.add_request(t, SamplingParams(max_tokens=max_tokens, ignore_eos=True),
                            request_id=rid)
        pending = []
    done, steps = {}, 0
    while (pending or eng.has_work()) and steps < 600:
        if pending and steps % arrive_every == 0:
            rid, t = pending.pop(0)
            eng.add_request(t, SamplingParams(max_tokens=max_tokens, ignore_eos=True),
                            request_id=rid)
        for o in eng.step():
            if o.finished:
                done[o.request_id] = list(o.output_token_ids)
        steps += 1
    return done


def _assert_greedy(cfg, W, prompts, done, tol):
    assert set(done) == set(prompts)
    for rid, t in prompts.items():
        gen = done[rid]
        logits = oracle.forward(cfg, W, t + gen)
        for i, tok in enumerate(gen):
            row = logits[len(t) - 1 + i]
            assert row[tok] >= row.max() - tol * row.std(), (rid, i)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=20)
    eng = LLMEngine(EngineConfig(
        model=d, device=device, dtype="float32", num_gpu_blocks=40, max_num_seqs=3,
        max_model_len=256, max_num_batched_tokens=24,  # prompts get chunked
        enable_graphs=False))
    prompts = {"p%d" % i: tokens(n, MIXED["vocab"], 50 + i)
               for i, n in enumerate([31, 5, 47, 12, 2])}
    done = _generate(eng, prompts, 12)
    assert all(len(g) == 12 for g in done.values())
    _assert_greedy(MIXED, W, prompts, done, 1e-3)
    assert eng.block_manager.num_free_blocks == eng.block_manager.num_blocks


def test_requests_arriving_under_a_tight_pool(tmp_path):
    d, W = model_dir(tmp_path, MIXED, seed=21)
    eng = LLMEngine(EngineConfig(
        model=d, device="cpu", dtype="float32", num_gpu_blocks=7, max_num_seqs=2,
        max_model_len=128, max_num_batched_tokens=16, enable_graphs=False))
    prompts = {"q%d" % i: tokens(n, MIXED["vocab"], 60 + i) for i, n in enumerate([30, 9, 21, 4])}
    done = _generate(eng, prompts, 10, arrive_every=3)
    _assert_greedy(MIXED, W, prompts, done, 1e-3)
    assert eng.block_manager.num_free_blocks == eng.block_manager.num_blocks


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graph_replays_match_oracle(tmp_path, dtype):
    cfg = OTHER["sixteens"]
    d, W = model_dir(tmp_path, cfg, seed=22)
    eng = LLMEngine(EngineConfig(
        model=d, device="cuda", dtype=dtype, num_gpu_blocks=40, max_num_seqs=4,
        max_model_len=256, max_num_batched_tokens=64, enable_graphs=True))
    prompts = {"g%d" % i: tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate([9, 20, 3])}
    done = _generate(eng, prompts, 24)
    assert all(len(g) == 24 for g in done.values())
    _assert_greedy(cfg, W, prompts, done, 1e-3 if dtype == "float32" else 0.1)


def test_preset_builds_and_generates():
    eng = LLMEngine(EngineConfig(
        model="vigonex-tiny", device="cpu", dtype="float32", num_gpu_blocks=16,
        max_num_seqs=2, max_model_len=64, enable_graphs=False))
    done = _generate(eng, {"a": tokens(9, 512, 1), "b": tokens(3, 512, 2)}, 5)
    assert all(len(g) == 5 for g in done.values())


# ---------------------------------------------------------------------------
# kernels one by one against the reference ops
# ---------------------------------------------------------------------------
def _close(got, want, dtype):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    scale = max(1.0, float(want.float().abs().max()))
    assert float((got.float().cpu() - want.float()).abs().max()) <= tol * scale


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C,S", [(24, 1), (256, 2), (1000, 4), (4096, 2), (64, 8)])
def test_kernel_stream_norm(dtype, C, S):
    g = torch.Generator().manual_seed(C)
    T = 9
    X = torch.randn(T, S, C, generator=g)
    gate = torch.randn(T, C, generator=g).to(dtype)
    mix, wr, rd = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    w = torch.rand(C, generator=g)
    for y in (torch.randn(T, C, generator=g).to(dtype), torch.randn(T, C, generator=g)):
        Xc, Xg = X.clone(), X.cuda()
        want = sops.hyper_mix_rmsnorm(Xc, y, gate, mix, wr, rd, w, 1e-6, dtype)
        got = sops.hyper_mix_rmsnorm(Xg, y.cuda(), gate.cuda(), mix.cuda(), wr.cuda(), rd.cuda(),
                                     w.cuda(), 1e-6, dtype)
        _close(got, want, dtype)
        _close(Xg, Xc, torch.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernel_activation_embedding_join(dtype):
    g = torch.Generator().manual_seed(9)
    for group, n, pad in ((8, 3, 0), (96, 12, 0), (5, 2, 0), (64, 4, 16)):
        gu = (2.0 * torch.randn(33, n * 2 * group + pad, generator=g)).to(dtype)[:, : n * 2 * group]
        rw = torch.rand(33, n, generator=g)
        for kw in (dict(alpha=1.702, limit=1.25, up_shift=1.0), dict(), dict(w_sigmoid=True)):
            _close(sops.glu_weighted(gu.cuda(), rw.cuda(), group, **kw),
                   sops.glu_weighted(gu, rw, group, **kw), dtype)
        _close(sops.glu_weighted(gu.cuda(), None, group), sops.glu_weighted(gu, None, group), dtype)
    from kubeai_amd.models.vigonex import sinusoid_frequencies
    table = torch.randn(50, 200, generator=g).to(dtype)
    ids = torch.randint(0, 50, (40,), generator=g, dtype=torch.int32)
    pos = torch.randint(0, 3000, (40,), generator=g, dtype=torch.int32)
    f = sinusoid_frequencies(200)
    got = sops.embed_sinusoid(ids.cuda(), table.cuda(), 2.5, pos.cuda(), f.cuda(), 2)
    want = sops.embed_sinusoid(ids, table, 2.5, pos, f, 2)
    assert float((got.cpu() - want).abs().max()) < (1e-5 if dtype == torch.float32 else 0.1)
    att_ = torch.randn(21, 2, 2, 3, 40, generator=g).to(dtype)
    out = torch.zeros(21, 6, 40, dtype=dtype)
    sops.diff_combine(att_, 0.6, 0.7, 1e-6, out)
    outg = torch.zeros(21, 6, 40, dtype=dtype, device="cuda")
    sops.diff_combine(att_.cuda(), 0.6, 0.7, 1e-6, outg)
    _close(outg, out, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,Dv", [(4, 64, 64), (2, 48, 48), (3, 10, 6), (1, 128, 128),
                                    (2, 16, 16), (1, 256, 256), (2, 96, 32)])
def test_kernel_delta_scan(dtype, H, D, Dv):
    lens, slots = [70, 1, 19, 1, 2], [2, 0, 3, -1, 1]
    starts = [0, 5, 0, 9, 33]
    parts = [_delta_inputs(n, H, D, Dv, 200 + i) for i, n in enumerate(lens)]
    wb, ab = parts[0][5], parts[0][6]
    cat = [torch.cat([p[j] for p in parts]).to(dtype) for j in range(5)]
    pos = [s + p for n, s in zip(lens, starts) for p in range(n)]
    g = torch.Generator().manual_seed(H)
    state = 0.5 * torch.randn(4, H, D, Dv, generator=g)
    sc, sg = state.clone(), state.cuda()
    scale = math.exp(-0.5)
    want = sops.diag_rank1_scan(*cat, wb, ab, sc, meta_of(list(zip(lens, slots)), pos, "cpu"), scale)
    got = sops.diag_rank1_scan(*[c.cuda() for c in cat], wb.cuda(), ab.cuda(), sg,
                               meta_of(list(zip(lens, slots)), pos, "cuda"), scale)
    tol = 3e-4 * max(1.0, float(want.abs().max()))
    assert float((got.cpu() - want).abs().max()) < tol
    assert float((sg.cpu() - sc).abs().max()) < 3e-4 * max(1.0, float(sc.abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("n", [127, 128, 129, 257, 1000])
def test_kernel_delta_scan_long_runs(n):
    H, D = 2, 64
    ins = _delta_inputs(n, H, D, D, n)
    scale = math.exp(-0.5)
    state = torch.zeros(2, H, D, D)
    want = sops.diag_rank1_scan(*ins, state.clone(), meta_of([(n, 0)], list(range(n)), "cpu"), scale)
    got = sops.diag_rank1_scan(*[x.cuda() for x in ins], state.cuda(),
                               meta_of([(n, 0)], list(range(n)), "cuda"), scale)
    assert float((got.cpu() - want).abs().max()) < 3e-4 * max(1.0, float(want.abs().max()))
