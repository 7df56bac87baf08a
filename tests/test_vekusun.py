"""Vekusun (latent attention with a query latent and learned sinks / latent
attention with a rotated shared key part and head gates / gated delta rule;
one norm feeding both sublayers; GELU or routed gated experts; a looped span
of layers) in the engine against the plain oracle in vekusun_oracle.py: every
mechanism alone, prompt vs token-by-token decoding, prompt portions down to
two tokens, unequal batches, reuse of freed cache blocks and state slots, keys
far back and at page borders (planted so that one score stands out), the
sink's share, first tokens, long decoding, other sizes, and greedy generation
through the engine's own scheduler. CPU runs use the torch reference ops; the
same cases run on the GPU kernels under the gpu marker, where the kernels are
also compared one by one with the reference ops.
"""
import json
import math
import os

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import vekusun_oracle as oracle
from kubeai_amd.engine import EngineConfig, LLMEngine, SamplingParams
from kubeai_amd.ops import seq as sops

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
GPU = [pytest.param("cuda", marks=pytest.mark.gpu)]

# base 40 over 12 dims with these constants: pairs 0 and 1 keep their
# frequency, pairs 2..4 are interpolated, pair 5 is divided by the factor
SCALING = {"factor": 3.0, "original": 48, "fast": 4.0, "slow": 0.5}

DENSE = {"kind": "dense", "ff": 40}


def moe(experts=5, top=2, ff=12):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


MOE = moe()


def lat1(heads=3, dim=6, vdim=4, rank=10, q_rank=14, scale=0.7, mlp=DENSE):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank,
                      "q_rank": q_rank, "scale": scale}}


def lat2(heads=2, dim=6, rot=12, vdim=10, rank=9, scale=0.5, base=40.0, scaling=SCALING,
         mlp=MOE):
    mx = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank,
          "scale": scale}
    if rot:
        mx["rot"] = {"base": base, "dims": rot}
        if scaling:
            mx["rot"]["scaling"] = scaling
    return {"type": "latent_attention_2", "mixer": mx, "mlp": mlp}


def delta(heads=4, kv=2, dim=10, vdim=6, conv=4, mlp=DENSE):
    return {"type": "delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}}


def config(layers, width=32, vocab=50, eps=1e-5, mult=0.7, cap=12.0, loop=None):
    cfg = {"architecture": "Vekusun", "vocab": vocab, "width": width,
           "norm": {"eps": eps}, "residual_mult": mult, "logit_softcap": cap,
           "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# layers 1..2 run twice: a delta layer and a rotated latent layer get two
# states / caches each; the loop does not start at layer 0
MIXED = config([lat1(), delta(), lat2(), lat1(heads=2, dim=4, vdim=8, rank=6, q_rank=5, mlp=MOE),
                delta(heads=2, kv=2, dim=16, vdim=16, conv=2, mlp=None)], loop=(1, 3, 2))


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
    g = torch.Generator().manual_seed(3000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_err(got, want):
    got = got.double().cpu().numpy() if isinstance(got, torch.Tensor) else got
    return np.abs(got - want).max(-1) / want.std()


def check(got, want, dtype="float32", loose=0.15):
    err = rel_err(got, want).max()
    # bf16: the widths here are tiny, so roundings do not average out
    assert err < (2e-4 if dtype == "float32" else loose), f"relative error {err:.3g}"


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


# ---------------------------------------------------------------------------
# mechanisms as functions: the product's ops against the oracle's
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("rot", [
    {"base": 40.0, "dims": 12, "scaling": SCALING},
    {"base": 40.0, "dims": 12},
    {"base": 50000.0, "dims": 64,
     "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
    {"base": 10.0, "dims": 2, "scaling": {"factor": 2.0, "original": 8, "fast": 2.0, "slow": 1.0}},
])
def test_ramped_frequencies(rot):
    from kubeai_amd.models.mixers import ramped_rotary_frequencies

    got, mult = ramped_rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    want, want_mult = oracle.ramped_frequencies(rot)
    assert np.abs(npy(got) / want - 1).max() < 1e-6
    assert abs(mult - want_mult) < 1e-12


def test_scaling_constants_cover_every_branch_of_the_ramp():
    f0, _ = oracle.ramped_frequencies({"base": 40.0, "dims": 12})
    f, mult = oracle.ramped_frequencies({"base": 40.0, "dims": 12, "scaling": SCALING})
    ratio = f / f0
    assert ratio[0] == 1.0 and ratio[1] == 1.0 and abs(ratio[-1] - 1 / 3) < 1e-12
    assert ((ratio[2:5] < 1.0) & (ratio[2:5] > 1 / 3)).all()
    assert mult > 1.0


@pytest.mark.parametrize("device", DEVICES)
def test_router_choice_and_weights(device):
    g = torch.Generator().manual_seed(1)
    z = torch.randn(70, 9, generator=g)
    z[3, 2] = z[3, 7] = 5.0  # equal scores: the lower index wins
    bias = torch.randn(9, generator=g) * 0.2
    W = {"r.router": np.eye(9), "r.correction": npy(bias)}
    for top in (1, 3, 9):
        dense, w, idx = sops.router_scores_topk(z.to(device), top, bias.to(device))
        want_idx, want_w = oracle.route(npy(z), W, "r.", {"router": {"top": top}})
        assert (idx.cpu().numpy() == want_idx).all()
        assert np.abs(npy(w) - want_w).max() < 1e-6
        # weights are the scores themselves: they do not sum to one unless all are chosen
        assert (abs(npy(w).sum(-1) - 1) < 1e-5).all() == (top == 9)
        d = npy(dense)
        assert (np.count_nonzero(d, axis=-1) == top).all()
        assert np.abs(np.take_along_axis(d, want_idx, -1) - want_w).max() < 1e-6
    # the correction steers the choice but not the weight
    z2 = torch.tensor([[2.0, 1.9, -1.0]])
    b2 = torch.tensor([0.0, 0.5, 0.0])
    _, w, idx = sops.router_scores_topk(z2.to(device), 1, b2.to(device))
    s = torch.softmax(z2, -1)
    assert idx.item() == 1 and abs(w.item() - s[0, 1].item()) < 1e-6
    _, w, idx = sops.router_scores_topk(z2.to(device), 1, None)
    assert idx.item() == 0


@pytest.mark.parametrize("device", DEVICES)
def test_scaled_add_norm_function(device):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 24, generator=g)
    a, b = torch.randn(5, 24, generator=g) * 3, torch.randn(5, 24, generator=g)
    sa, sb, w = (torch.randn(24, generator=g) for _ in range(3))
    extra, row = torch.randn(5, 24, generator=g), torch.randn(24, generator=g)
    dev = lambda t: t.to(device)
    res = dev(x.clone())
    h = sops.scaled_add_rmsnorm(res, dev(a), dev(sa), dev(b), dev(sb), 0.3, dev(extra),
                                dev(row), dev(w), 1e-3, torch.float32)
    x2 = npy(x) + 0.3 * (npy(a) * npy(sa) + npy(b) * npy(sb)) + npy(extra) + npy(row)
    assert np.abs(npy(res) - x2).max() < 1e-5
    assert np.abs(npy(h) - oracle.rms_norm(x2, npy(w), 1e-3)).max() < 1e-5
    # one branch, nothing else; then the norm alone leaves the residual as it is
    res = dev(x.clone())
    h = sops.scaled_add_rmsnorm(res, dev(a), dev(sa), None, None, 1.0, None, None, dev(w),
                                1e-3, torch.float32)
    x3 = npy(x) + npy(a) * npy(sa)
    assert np.abs(npy(res) - x3).max() < 1e-5
    h = sops.scaled_add_rmsnorm(res, None, None, None, None, 1.0, None, None, dev(w), 1e-3,
                                torch.float32)
    assert np.abs(npy(res) - x3).max() < 1e-5
    assert np.abs(npy(h) - oracle.rms_norm(x3, npy(w), 1e-3)).max() < 1e-5


def _delta_inputs(T, H, G, D, Dv, seed):
    g = torch.Generator().manual_seed(seed)
    q, k = torch.randn(T, G, D, generator=g), torch.randn(T, G, D, generator=g)
    v = torch.randn(T, H, Dv, generator=g)
    b, a = torch.randn(T, H, generator=g) * 2, torch.randn(T, H, generator=g) * 2
    a_log, dt = torch.randn(H, generator=g), torch.randn(H, generator=g)
    return q, k, v, b, a, a_log, dt


def _delta_want(q, k, v, b, a, a_log, dt):
    T, G, D = q.shape
    H = v.shape[1]
    qn, kn = npy(q), npy(k)
    qn = qn / np.sqrt((qn * qn).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    kn = kn / np.sqrt((kn * kn).sum(-1, keepdims=True) + 1e-6)
    beta = oracle.sigmoid(npy(b))
    dec = np.exp(-np.exp(npy(a_log)) * oracle.softplus(npy(a) + npy(dt)))
    return np.stack([oracle.delta_recurrence(qn[:, h // (H // G)], kn[:, h // (H // G)],
                                             npy(v)[:, h], beta[:, h], dec[:, h])
                     for h in range(H)], axis=1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 10, 6), (2, 2, 16, 16), (3, 1, 32, 20),
                                      (1, 1, 3, 70)])
def test_delta_scan_function_and_carried_state(device, H, G, D, Dv):
    """One run in one call, against the same tokens cut into three calls that
    carry the state in a slot which held another sequence before."""
    T = 23
    q, k, v, b, a, a_log, dt = _delta_inputs(T, H, G, D, Dv, 5)
    want = _delta_want(q, k, v, b, a, a_log, dt)
    dev = lambda t: t.to(device)
    state = torch.randn(3, H, D, Dv).to(device)  # stale contents of the slots
    for cuts in ([T], [9, 1, 13], [1] * T):
        got, at = [], 0
        for n in cuts:
            meta = sops.SeqMeta.build([(n, 1)], torch.arange(at, at + n, dtype=torch.int32).to(device),
                                      device)
            got.append(sops.gated_delta_scan(
                dev(q[at : at + n]), dev(k[at : at + n]), dev(v[at : at + n]),
                dev(b[at : at + n]), dev(a[at : at + n]), dev(a_log), dev(dt), state, meta))
            at += n
        assert np.abs(npy(torch.cat(got)) - want).max() < 2e-5


@pytest.mark.parametrize("device", DEVICES)
def test_delta_scan_long_runs_and_unequal_batch(device):
    """A 700-token run (cut into parallel segments on the GPU) beside a short
    one and a single token that continues a stored state."""
    H, G, D, Dv = 2, 1, 16, 20
    lens = [700, 37, 1]
    ins = [_delta_inputs(n, H, G, D, Dv, 6 + i) for i, n in enumerate(lens)]
    want = [_delta_want(*x) for x in ins]
    dev = lambda t: t.to(device)
    state = torch.zeros(4, H, D, Dv).to(device)
    # the third run continues sequence 1 of `ins` after its 36 first tokens
    x1 = ins[1]
    meta = sops.SeqMeta.build([(36, 2)], torch.arange(36, dtype=torch.int32).to(device), device)
    sops.gated_delta_scan(*(dev(t[:36]) for t in x1[:5]), dev(x1[5]), dev(x1[6]), state, meta)
    pos = torch.cat([torch.arange(700), torch.arange(37), torch.tensor([36])]).int().to(device)
    meta = sops.SeqMeta.build([(700, 0), (37, 3), (1, 2)], pos, device)
    cat = [torch.cat([ins[0][j], ins[1][j], ins[1][j][36:37]]) for j in range(5)]
    got = npy(sops.gated_delta_scan(*(dev(t) for t in cat), dev(ins[0][5]), dev(ins[0][6]),
                                    state, meta))
    # all runs share a_log / dt_bias of ins[0] in this call: recompute the others
    w1 = _delta_want(*ins[1][:5], ins[0][5], ins[0][6])
    assert np.abs(got[:700] - want[0]).max() < 5e-5
    assert np.abs(got[700:737] - w1).max() < 5e-5
    # the single token continues a state made with ins[1]'s own constants
    w_own = _delta_want(*ins[1])
    state2 = torch.zeros(4, H, D, Dv).to(device)
    meta = sops.SeqMeta.build([(36, 2)], torch.arange(36, dtype=torch.int32).to(device), device)
    sops.gated_delta_scan(*(dev(t[:36]) for t in x1[:5]), dev(x1[5]), dev(x1[6]), state2, meta)
    meta = sops.SeqMeta.build([(1, 2)], torch.tensor([36], dtype=torch.int32).to(device), device)
    one = sops.gated_delta_scan(*(dev(t[36:37]) for t in x1[:5]), dev(x1[5]), dev(x1[6]),
                                state2, meta)
    assert np.abs(npy(one)[0] - w_own[36]).max() < 5e-5


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_overwrites_what_a_key_holds(device):
    """With beta = 1 and no decay, writing v2 at a key that holds v1 leaves
    v2 alone: the rule corrects, it does not accumulate."""
    D, Dv = 16, 16
    k = torch.zeros(3, 1, D)
    k[:, 0, 2] = 5.0
    v = torch.zeros(3, 1, Dv)
    v[0, 0, 1], v[1, 0, 3], v[2, 0, 3] = 4.0, -2.0, -2.0
    q = k.clone()
    big = torch.full((3, 1), 30.0)   # sigmoid -> 1
    a = torch.full((3, 1), -30.0)    # softplus -> 0: decay 1
    meta = sops.SeqMeta.build([(3, 0)], torch.arange(3, dtype=torch.int32).to(device), device)
    state = torch.zeros(1, 1, D, Dv).to(device)
    o = npy(sops.gated_delta_scan(q.to(device), k.to(device), v.to(device), big.to(device),
                                  a.to(device), torch.zeros(1).to(device),
                                  torch.zeros(1).to(device), state, meta)) * D ** 0.5
    assert abs(o[0, 0, 1] - 4.0) < 1e-4
    assert abs(o[1, 0, 1]) < 1e-4 and abs(o[1, 0, 3] + 2.0) < 1e-4
    assert abs(o[2, 0, 3] + 2.0) < 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_conv_silu_and_carried_tail(device):
    g = torch.Generator().manual_seed(7)
    C, taps, T = 9, 4, 12
    x, w = torch.randn(T, C, generator=g), torch.randn(C, taps, generator=g)
    want = oracle.short_conv_silu(npy(x), npy(w))
    for cuts in ([T], [1, 2, 5, 4], [1] * T):
        tails = torch.randn(2, taps - 1, C).to(device)  # stale
        got, at = [], 0
        for n in cuts:
            meta = sops.SeqMeta.build([(n, 1)], torch.arange(at, at + n, dtype=torch.int32).to(device),
                                      device)
            got.append(sops.causal_conv(x[at : at + n].to(device), w.to(device), tails, meta,
                                        False, act="silu"))
            at += n
        assert np.abs(npy(torch.cat(got)) - want).max() < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,R,half", [(2, 9, 6), (4, 64, 8), (1, 5, 1)])
def test_latent_rows_with_rotated_part(device, H, R, half):
    g = torch.Generator().manual_seed(8)
    T, bs = 21, 16
    rot = {"base": 40.0, "dims": 2 * half, "scaling": SCALING}
    f, mult = oracle.ramped_frequencies(rot)
    x = torch.randn(T, R + 2 * half, generator=g)
    qfull = torch.randn(T, H, 7 + 2 * half, generator=g)
    w = torch.randn(R, generator=g)
    pos = torch.randint(0, 900, (T,), generator=g).int()
    cache = torch.zeros(3, 1, bs, R + 2 * half)
    slots = torch.randperm(3 * bs, generator=g)[:T]
    slots[4] = -1
    ql = torch.zeros(T, H, R + 2 * half)
    cache, ql = cache.to(device), ql.to(device)
    sops.latent_rope_to_cache(x.to(device), w.to(device), 1e-4, qfull.to(device)[..., 7:],
                              ql[..., R:], pos.to(device),
                              torch.tensor(f, dtype=torch.float32).to(device), mult, cache,
                              slots.to(device))
    want = np.concatenate([oracle.rms_norm(npy(x[:, :R]), npy(w), 1e-4),
                           oracle.rotate_pairs(npy(x[:, R:]), pos.numpy(), f, mult)], -1)
    flat = npy(cache).reshape(-1, R + 2 * half)
    for t in range(T):
        if slots[t] >= 0:
            assert np.abs(flat[slots[t]] - want[t]).max() < 2e-4
    assert np.count_nonzero(np.abs(flat).sum(-1)) == T - 1
    wq = oracle.rotate_pairs(npy(qfull[..., 7:]), pos.numpy(), f, mult)
    assert np.abs(npy(ql[..., R:]) - wq).max() < 2e-4
    assert np.abs(npy(ql[..., :R])).max() == 0


# ---------------------------------------------------------------------------
# every mechanism alone, in the engine
# ---------------------------------------------------------------------------
SINGLE = {
    "query_latent_no_ff": config([lat1(mlp=None)]),
    "query_latent_one_head": config([lat1(heads=1, dim=16, vdim=3, rank=5, q_rank=3)]),
    "query_latent_equal_sizes": config([lat1(heads=2, dim=8, vdim=8, rank=8, q_rank=8)]),
    "rotated_latent_no_ff": config([lat2(mlp=None)]),
    "rotated_latent_no_scaling": config([lat2(scaling=None, mlp=DENSE)]),
    "rotated_latent_one_pair": config([lat2(heads=3, dim=4, rot=2, vdim=2, rank=7, mlp=DENSE)]),
    "rotated_latent_without_a_rotated_part": config([lat2(rot=0, mlp=DENSE)]),
    "rotated_latent_one_head": config([lat2(heads=1, dim=8, rot=4, vdim=3, rank=5, mlp=None)]),
    "delta_no_ff": config([delta(mlp=None)]),
    "delta_every_head_its_own_key": config([delta(heads=3, kv=3, dim=8, vdim=8)]),
    "delta_one_key_head": config([delta(heads=4, kv=1, dim=16, vdim=4, conv=2)]),
    "delta_one_tap": config([delta(conv=1)]),
    "experts_top_one": config([lat1(mlp=moe(experts=4, top=1))]),
    "experts_all_chosen": config([delta(mlp=moe(experts=3, top=3))]),
    "one_expert": config([lat2(mlp=moe(experts=1, top=1))]),
    "no_multiplier_no_cap": config([lat1(), delta()], mult=1.0, cap=0.0),
    "loop_of_everything": config([delta(), lat2()], loop=(0, 2, 3)),
    "loop_once": config([lat1(), delta()], loop=(1, 2, 1)),
    "loop_of_the_last_layer": config([lat1(), lat2(), delta()], loop=(2, 3, 2), mult=0.4),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_whole_prompt(tmp_path, device, name):
    cfg = SINGLE[name]
    d, W = model_dir(tmp_path, cfg, seed=3)
    toks = tokens(37, cfg["vocab"], 1)
    want = oracle.forward(cfg, W, toks)
    check(replay(engine(d, device), "a", toks, [len(toks)]), want)
    check(replay(engine(d, device), "b", toks, [5, 1]), want)


@pytest.mark.parametrize("device", DEVICES)
def test_layers_match_after_every_layer_run(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=4)
    toks = tokens(29, MIXED["vocab"], 2)
    layers = []
    oracle.forward(MIXED, W, toks, capture=layers)
    eng = engine(d, device)
    eng.runner.model.capture_layers = []
    replay(eng, "a", toks, [len(toks)])
    got = torch.stack(eng.runner.model.capture_layers)[:, : len(toks)]
    assert got.shape[0] == len(layers) == 7  # 1 + 2 * 2 + 2 layer runs
    for i, want in enumerate(layers):
        check(got[i], want)


# ---------------------------------------------------------------------------
# prompt vs decoding, portions, first tokens
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2, 5], [7, 1, 1, 4, 1], [16, 1], [11, 13]])
def test_portions_and_token_by_token(tmp_path, device, cuts):
    d, W = model_dir(tmp_path, MIXED, seed=5)
    toks = tokens(45, MIXED["vocab"], 3)
    check(replay(engine(d, device), "a", toks, cuts), oracle.forward(MIXED, W, toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("n", [1, 2, 3])
def test_first_tokens(tmp_path, device, n):
    d, W = model_dir(tmp_path, MIXED, seed=6)
    toks = tokens(n, MIXED["vocab"], 4)
    want = oracle.forward(MIXED, W, toks)
    check(replay(engine(d, device), "a", toks, [n]), want)
    check(replay(engine(d, device), "b", toks, [1]), want)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(tmp_path, device):
    d, W = model_dir(tmp_path, MIXED, seed=7)
    toks = tokens(150, MIXED["vocab"], 5)
    check(replay(engine(d, device), "a", toks, [9, 1]), oracle.forward(MIXED, W, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_long_prompt_in_one_step_and_routed_path(tmp_path, device):
    """Steps above the dense-expert threshold gather tokens per expert, and
    the delta scan cuts the run into segments (GPU): both against the oracle."""
    from kubeai_amd.models.mixers import RoutedGatedMoE

    cfg = config([delta(heads=2, kv=1, dim=16, vdim=12, mlp=moe(experts=6, top=2)),
                  lat2(mlp=moe(experts=3, top=1))])
    d, W = model_dir(tmp_path, cfg, seed=8)
    toks = tokens(RoutedGatedMoE.DENSE_MAX_TOKENS + 75, cfg["vocab"], 6)
    want = oracle.forward(cfg, W, toks)
    check(replay(engine(d, device), "a", toks, [len(toks)]), want)
    check(replay(engine(d, device), "b", toks, [300, 2, 1]), want)


# sizes in multiples of 16: bf16 prompt portions take the matrix-core kernels.
# Every expert is chosen, so that no rounding can flip a routing decision.
SIXTEENS = config(
    [lat1(heads=4, dim=16, vdim=32, rank=48, q_rank=32, scale=0.25,
          mlp=moe(experts=3, top=3, ff=32)),
     lat2(heads=2, dim=32, rot=16, vdim=16, rank=64, scale=0.15, mlp=DENSE),
     delta(heads=4, kv=2, dim=32, vdim=16, conv=3, mlp=moe(experts=2, top=2, ff=16))],
    width=64, vocab=80, loop=(0, 2, 2))


# odd sizes: the generic kernels. With key sizes of 6 and 10 the reference ops
# on the CPU land at 0.2 in bf16 for this model (0.06 for SIXTEENS).
ODD = config([lat1(), delta(), lat2(mlp=moe(experts=3, top=3)), delta(mlp=None)],
             loop=(1, 3, 2))


@pytest.mark.parametrize("device", GPU)
@pytest.mark.parametrize("name", ["odd_sizes", "sixteens"])
def test_bfloat16_serving_precision(tmp_path, device, name):
    cfg, loose = {"odd_sizes": (ODD, 0.4), "sixteens": (SIXTEENS, 0.15)}[name]
    d, W = model_dir(tmp_path, cfg, seed=9)
    toks = tokens(70, cfg["vocab"], 7)
    want = oracle.forward(cfg, W, toks)
    check(replay(engine(d, device, "bfloat16"), "a", toks, [len(toks)]), want, "bfloat16", loose)
    check(replay(engine(d, device, "bfloat16"), "b", toks, [33, 2, 1]), want, "bfloat16", loose)
    check(replay(engine(d, device, "float32"), "c", toks, [33, 2, 1]), want)


# ---------------------------------------------------------------------------
# batches, reuse of blocks and slots
# ---------------------------------------------------------------------------
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


# ---------------------------------------------------------------------------
# keys far back and at page borders, the sink: one score made to stand out
# ---------------------------------------------------------------------------
def _planted(device, q_pos, key_pos, sink, rot=0, block=16, decode=False,
             dtype=torch.float32, dims=(2, 8), boost=40.0):
    """Latent-style attention over rows that serve as keys and values (the
    values are the leading R columns of rows R + rot wide): only key_pos has
    a large aligned entry. Returns (got, want) for the query at q_pos."""
    H, R = dims
    T = q_pos + 1
    rows = torch.zeros(T, R + rot)
    rows[key_pos, 0] = boost
    rows[key_pos, 1:R] = 7.0
    if rot:
        rows[key_pos, R] = 3.0   # the rotated part joins the score only
    q = torch.zeros(T, H, R + rot)
    q[:, :, 0] = 1.0
    if rot:
        q[:, :, R] = 0.5
    s = npy(q[:, 0]) @ npy(rows).T
    sink_t = None if sink is None else torch.tensor([sink, sink - 1.0][:H])
    want = [(oracle.causal_softmax(s, None if sink is None else float(sink_t[h]))
             @ npy(rows[:, :R]))[q_pos] for h in range(H)]
    nblk = (T + block - 1) // block
    perm = torch.randperm(nblk + 3, generator=torch.Generator().manual_seed(T)).tolist()
    table = torch.tensor([perm[:nblk]], dtype=torch.int32)
    cache = torch.zeros(nblk + 3, 1, block, R + rot)
    tp = torch.arange(T)
    cache[table[0][tp // block].long(), 0, tp % block] = rows
    if decode:
        runs, positions, qq = [(1, 0)], torch.tensor([q_pos], dtype=torch.int32), q[q_pos:]
    else:
        lo = max(0, q_pos - 20)
        runs, positions = [(q_pos + 1 - lo, 0)], torch.arange(lo, q_pos + 1, dtype=torch.int32)
        qq = q[lo:]
    meta = sops.SeqMeta.build(runs, positions.to(device), device,
                              block_tables=table.to(device))
    out = torch.zeros(qq.shape[0], H, R, device=device, dtype=dtype)
    cache = cache.to(device, dtype)
    sops.masked_paged_attention(qq.to(device, dtype).contiguous(), cache,
                                cache[..., :R] if rot else cache, meta, 1.0, out,
                                sink=None if sink is None else sink_t.to(device))
    return npy(out[-1].float()), np.stack(want)


FAR = [(99, 90), (47, 32), (47, 31), (48, 47), (700, 3), (1029, 0), (5, 0), (15, 15), (16, 16)]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("rot", [0, 4])
@pytest.mark.parametrize("q_pos,key_pos", FAR)
def test_planted_key_far_back_and_at_page_borders(device, decode, rot, q_pos, key_pos):
    got, want = _planted(device, q_pos, key_pos, sink=1.5, rot=rot, decode=decode)
    assert abs(want[0, 1] - 7.0) < 1e-6  # the planted key takes all the weight
    assert np.abs(got - want).max() < 1e-4


@pytest.mark.parametrize("device", GPU)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("rot", [0, 16])
@pytest.mark.parametrize("q_pos,key_pos", FAR)
def test_planted_key_matrix_core_kernels(device, decode, rot, q_pos, key_pos):
    got, want = _planted(device, q_pos, key_pos, sink=1.5, rot=rot, decode=decode,
                         dtype=torch.bfloat16, dims=(2, 32), boost=48.0)
    assert np.abs(got - want).max() < 0.05
    # 16 heads on one row: the grouped decode kernel
    got, want = _planted(device, q_pos, key_pos, sink=None, rot=rot, decode=decode,
                         dtype=torch.bfloat16, dims=(1, 32), boost=48.0)
    assert np.abs(got - want).max() < 0.05


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sink", [-30.0, 0.0, 3.0, 38.0])
def test_sink_takes_its_share(device, sink):
    """Key score 40 * 1 against sink scores sink and sink - 1 on the two
    heads: the output shrinks by exactly the sink's share, which differs
    between the heads; the sink is not scaled with the keys' scores."""
    for decode in (False, True):
        got, want = _planted(device, 12, 12, sink=sink, decode=decode)
        assert np.abs(got - want).max() < 1e-4
        share = 1.0 / (1.0 + math.exp(sink - 40.0))
        assert abs(got[0, 1] - 7.0 * share) < 1e-3
        if sink > 30:
            assert got[1, 1] > got[0, 1] + 0.5  # the second head's sink is weaker
    got, want = _planted(device, 12, 12, sink=None)
    assert abs(got[0, 1] - 7.0) < 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_far_token_reaches_logits(tmp_path, device):
    """Changing token 2 changes the logits 300 tokens later as the oracle
    says: through the cached latents, and through the delta state alone."""
    for n, cfg in enumerate([config([lat1(scale=2.0, mlp=None), lat2(scale=1.5, mlp=None)]),
                             config([delta(heads=2, kv=1, dim=64, vdim=8, mlp=None)])]):
        W = oracle.random_weights(cfg, 14 + n)
        if n == 1:  # slow decay and a wide key space, so that the state remembers
            W["l0.mix.A_log"] = torch.full_like(W["l0.mix.A_log"], -6.0)
        d, W = model_dir(tmp_path, cfg, seed=14 + n, W=W)
        a = tokens(300, cfg["vocab"], 31)
        b = list(a)
        b[2] = (a[2] + 1) % cfg["vocab"]
        eng = engine(d, device)
        ga = npy(replay(eng, "a", a, [250, 3, 1])[-1])
        gb = npy(replay(eng, "b", b, [250, 3, 1])[-1])
        wa, wb = oracle.forward(cfg, W, a)[-1], oracle.forward(cfg, W, b)[-1]
        assert np.abs(wa - wb).max() > 1e-4 * wa.std()
        assert np.abs((ga - gb) - (wa - wb)).max() / wa.std() < 2e-4


# ---------------------------------------------------------------------------
# other sizes and orders
# ---------------------------------------------------------------------------
OTHER = {
    "delta_first_latents_after": config(
        [delta(heads=6, kv=3, dim=4, vdim=2, conv=3), lat2(heads=5, dim=2, rot=6, vdim=2, rank=12),
         lat1(heads=1, dim=2, vdim=20, rank=12, q_rank=40, mlp=MOE)], width=24, vocab=33,
        loop=(0, 1, 2)),
    "wide_rotation_small_latent": config(
        [lat2(heads=2, dim=2, rot=20, vdim=6, rank=3, base=7.0, scale=1.3,
              scaling={"factor": 2.0, "original": 20, "fast": 3.0, "slow": 0.5}),
         lat2(heads=8, dim=4, rot=2, vdim=2, rank=33, mlp=DENSE)], width=16, eps=1e-3),
    "wide_experts": config([lat1(mlp=moe(experts=7, top=5, ff=30)),
                            delta(mlp=moe(experts=2, top=1, ff=50))], width=48, mult=1.5),
    "no_loop_entry": config([delta(), lat1()], width=40, vocab=70),
    "loop_four_times": config([lat1(), delta(conv=2)], loop=(0, 1, 4), cap=3.0),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_sizes(tmp_path, device, name):
    cfg = OTHER[name]
    d, W = model_dir(tmp_path, cfg, seed=15)
    toks = tokens(40, cfg["vocab"], 32)
    check(replay(engine(d, device), "a", toks, [13, 2, 1]), oracle.forward(cfg, W, toks))


def test_unconsumed_and_missing_tensors_are_errors(tmp_path):
    cfg = config([lat1()])
    W = oracle.random_weights(cfg, 16)
    W["l0.mix.extra"] = torch.zeros(3).bfloat16()
    d, _ = model_dir(tmp_path, cfg, seed=16, W=W)
    with pytest.raises(ValueError, match="not consumed"):
        engine(d, "cpu")
    W = oracle.random_weights(cfg, 17)
    del W["l0.mix.sink"]
    d, _ = model_dir(tmp_path, cfg, seed=17, W=W)
    with pytest.raises(ValueError, match="sink"):
        engine(d, "cpu")


def test_loop_must_fit_the_layers(tmp_path):
    cfg = config([lat1(), delta()], loop=(1, 3, 2))
    d, _ = model_dir(tmp_path, cfg, seed=18,
                     W=oracle.random_weights(config([lat1(), delta()], loop=(1, 2, 2)), 18))
    with pytest.raises(ValueError, match="loop"):
        engine(d, "cpu")


def test_every_pass_has_its_own_cache_and_state(tmp_path):
    cfg = config([delta(), lat2()], loop=(0, 2, 3))
    d, _ = model_dir(tmp_path, cfg, seed=19)
    eng = engine(d, "cpu")
    r = eng.runner
    assert len(r.kv_caches) == 6 and len(r.states) == 6
    assert sum(c is not None for c in r.kv_caches) == 3
    assert sum("s" in s for s in r.states) == 3
    rows = [c[0].shape[-1] for c in r.kv_caches if c is not None]
    assert rows == [9 + 12] * 3  # latent + rotated key part, nothing per head


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


def test_preemption_and_abort_keep_cache_and_state_consistent(tmp_path):
    d, W = model_dir(tmp_path, MIXED, seed=21)
    eng = LLMEngine(EngineConfig(
        model=d, device="cpu", dtype="float32", num_gpu_blocks=6, max_num_seqs=3,
        max_model_len=128, max_num_batched_tokens=64))  # tight pool: preemption
    prompts = {"q%d" % i: tokens(30, MIXED["vocab"], 70 + i) for i in range(3)}
    for rid, t in prompts.items():
        eng.add_request(t, SamplingParams(max_tokens=20, ignore_eos=True), request_id=rid)
    done, steps = {}, 0
    while eng.has_work() and steps < 600:
        if steps == 3:
            eng.abort_request("q1")
        for o in eng.step():
            if o.finished:
                done[o.request_id] = list(o.output_token_ids)
        steps += 1
    _assert_greedy(MIXED, W, {r: prompts[r] for r in ("q0", "q2")},
                   {r: done[r] for r in ("q0", "q2")}, 1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graph_replays_match_oracle(tmp_path, dtype):
    """Pure-decode steps replay a captured graph; prompt portions of later
    arrivals run eagerly between replays. Every generated token is checked."""
    cfg = MIXED if dtype == "float32" else SIXTEENS
    d, W = model_dir(tmp_path, cfg, seed=22)
    eng = LLMEngine(EngineConfig(
        model=d, device="cuda", dtype=dtype, num_gpu_blocks=64, max_num_seqs=6,
        max_model_len=512, max_num_batched_tokens=64, enable_graphs=True))
    prompts = {"g%d" % i: tokens(n, cfg["vocab"], 90 + i)
               for i, n in enumerate([9, 33, 4, 70, 18, 2, 25])}
    done = _generate(eng, prompts, 24, arrive_every=5)
    assert eng.runner._graphs, "no decode graph was captured"
    _assert_greedy(cfg, W, prompts, done, 1e-3 if dtype == "float32" else 0.25)


def test_preset_builds_and_generates():
    eng = LLMEngine(EngineConfig(model="vekusun-tiny", device="cpu", dtype="float32",
                                 num_gpu_blocks=16, max_num_seqs=2, max_model_len=128))
    eng.add_request(tokens(9, 512, 1), SamplingParams(max_tokens=4, ignore_eos=True),
                    request_id="r")
    out = []
    while eng.has_work():
        out += [o for o in eng.step() if o.finished]
    assert len(out) == 1 and len(out[0].output_token_ids) == 4


# ---------------------------------------------------------------------------
# kernels one by one against the reference ops (GPU)
# ---------------------------------------------------------------------------
def _close(got, want, dtype):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    scale = max(1.0, float(want.abs().max()))
    assert float((got.float().cpu() - want.float()).abs().max()) <= tol * scale


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C", [24, 256, 1000])
def test_kernel_scaled_add_norm(dtype, C):
    g = torch.Generator().manual_seed(C)
    T = 7
    x = torch.randn(T, C, generator=g)
    a, b = torch.randn(T, C, generator=g).to(dtype), torch.randn(T, C, generator=g)
    sa, sb, w, row = (torch.randn(C, generator=g) for _ in range(4))
    extra = torch.randn(T, C, generator=g)
    for bb in (b.to(dtype), b):  # second branch in the serving dtype, or fp32
        r_ref, r_gpu = x.clone(), x.clone().cuda()
        want = sops.scaled_add_rmsnorm(r_ref, a, sa, bb, sb, 0.5, extra, row, w, 1e-5, dtype)
        got = sops.scaled_add_rmsnorm(r_gpu, a.cuda(), sa.cuda(), bb.cuda(), sb.cuda(), 0.5,
                                      extra.cuda(), row.cuda(), w.cuda(), 1e-5, dtype)
        _close(r_gpu, r_ref, torch.float32)
        _close(got, want, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernel_elementwise_and_routing(dtype):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(37, 40, generator=g) * 3).to(dtype)
    _close(sops.gelu(x.cuda()), sops.gelu(x), dtype)
    _close(sops.gelu(x[:, :39].contiguous().cuda()), sops.gelu(x[:, :39].contiguous()), dtype)
    wide = (torch.randn(11, 64, generator=g)).to(dtype)
    w = torch.randn(24, generator=g)
    _close(sops.rmsnorm_rows(wide.cuda()[:, 8:32], w.cuda(), 1e-5),
           sops.rmsnorm_rows(wide[:, 8:32], w, 1e-5), dtype)
    lg = torch.randn(5, 33, generator=g) * 20
    _close(sops.tanh_cap(lg.clone().cuda(), 7.0), sops.tanh_cap(lg.clone(), 7.0), torch.float32)
    gu = torch.randn(19, 3 * 2 * 8, generator=g).to(dtype)
    rw = torch.rand(19, 3, generator=g)
    _close(sops.silu_mul_weighted(gu.cuda(), rw.cuda(), 8), sops.silu_mul_weighted(gu, rw, 8),
           dtype)
    _close(sops.silu_mul_weighted(gu[:, :16].contiguous().cuda(), rw.cuda()[:, 1:2], 8),
           sops.silu_mul_weighted(gu[:, :16].contiguous(), rw[:, 1:2], 8), dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,A,B,pad", [(1, 1, 16, 16, 0), (37, 3, 32, 48, 16), (70, 2, 192, 16, 4),
                                         (9, 4, 10, 6, 3), (130, 8, 64, 64, 16)])
def test_kernel_head_linear_on_slices_with_head_gate(dtype, T, H, A, B, pad):
    g = torch.Generator().manual_seed(T)
    xw = torch.randn(T, H, A + pad, generator=g).to(dtype)
    w = (torch.randn(H, B, A, generator=g) * A ** -0.5).to(dtype)
    gate = torch.randn(T, H + 3, generator=g).to(dtype)
    yw_ref = torch.zeros(T, H, B + pad, dtype=dtype)
    yw = yw_ref.clone().cuda()
    sops.head_linear(xw[..., :A], w, gate=gate[:, 3:], out=yw_ref[..., pad:])
    xg = xw.cuda()
    sops.head_linear(xg[..., :A], w.cuda(), gate=gate.cuda()[:, 3:], out=yw[..., pad:])
    _close(yw, yw_ref, dtype)
    _close(sops.head_linear(xg[..., :A], w.cuda()), sops.head_linear(xw[..., :A], w), dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,R,rot", [(4, 10, 6), (8, 64, 16), (16, 128, 64), (2, 32, 0),
                                     (16, 48, 16), (16, 96, 48), (8, 192, 64), (4, 256, 16)])
def test_kernel_attention_over_shared_rows_with_sinks(dtype, H, R, rot):
    g = torch.Generator().manual_seed(H)
    bs, nblk = 16, 12
    lens = [(40, 100), (1, 77), (9, 9), (1, 1)]  # (run length, sequence length)
    cache = (torch.randn(nblk * 4, 1, bs, R + rot, generator=g) * 0.5).to(dtype)
    tables = torch.stack([torch.randperm(nblk * 4, generator=g)[:nblk] for _ in lens]).int()
    pos = torch.cat([torch.arange(L - n, L) for n, L in lens]).int()
    T = int(pos.numel())
    q = (torch.randn(T, H, R + rot, generator=g) * 0.5).to(dtype)
    sink = torch.randn(H, generator=g)
    for decode_only in (False, True):
        if decode_only:
            runs, p, qq, tb = [(1, 0)] * 3, torch.tensor([99, 76, 0]).int(), q[:3], tables[:3]
        else:
            runs, p, qq, tb = [(n, 0) for n, _ in lens], pos, q, tables
        outs = []
        for dev in ("cpu", "cuda"):
            meta = sops.SeqMeta.build(runs, p.to(dev), dev, block_tables=tb.to(dev))
            c = cache.to(dev)
            out = torch.zeros(qq.shape[0], H, R, dtype=dtype, device=dev)
            sops.masked_paged_attention(qq.to(dev), c, c[..., :R] if rot else c, meta,
                                        R ** -0.5, out, sink=sink.to(dev))
            outs.append(out)
        _close(outs[1], outs[0].cpu(), dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [127, 128, 129, 200, 256, 257, 513])
def test_kernel_scans_at_segment_borders(n):
    """Run lengths around the sizes at which the scans start to cut a run
    into parallel segments: the delta rule and the linear-attention scan."""
    H, G, D, Dv = 2, 1, 16, 8
    ins = _delta_inputs(n, H, G, D, Dv, n)
    want = _delta_want(*ins)
    pos = torch.arange(n, dtype=torch.int32).cuda()
    meta = sops.SeqMeta.build([(n, 0)], pos, "cuda")
    state = torch.zeros(1, H, D, Dv).cuda()
    got = sops.gated_delta_scan(*(t.cuda() for t in ins), state, meta)
    assert np.abs(npy(got) - want).max() < 5e-5
    g = torch.Generator().manual_seed(n)
    q, k = (torch.randn(n, H, D, generator=g) * 0.3 for _ in range(2))
    v = torch.randn(n, H, Dv, generator=g)
    decay = torch.tensor([0.9, 0.97])
    res = []
    for dev in ("cpu", "cuda"):
        st = torch.zeros(1, H, D, Dv).to(dev)
        m = sops.SeqMeta.build([(n, 0)], pos.to(dev), dev)
        res.append(sops.linear_attn_scan(q.to(dev), k.to(dev), v.to(dev), decay.to(dev), None,
                                         st, m).cpu())
    assert float((res[0] - res[1]).abs().max()) < 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 32, 16), (2, 1, 128, 40), (3, 3, 10, 6),
                                      (8, 4, 64, 64), (2, 1, 64, 8), (2, 1, 48, 24),
                                      (1, 1, 80, 100), (2, 2, 16, 300), (1, 1, 200, 260),
                                      (2, 1, 24, 70)])
def test_kernel_delta_scan(dtype, H, G, D, Dv):
    """Register-state and LDS-state kernels, plain and segment-parallel runs,
    inputs as strided column views of one projection, against the reference."""
    lens = [(600, 0), (1, 2), (70, 1), (3, -1)]
    T = sum(n for n, _ in lens)
    g = torch.Generator().manual_seed(D)
    nqk, nv = G * D, H * Dv
    proj = torch.randn(T, 2 * nqk + nv + 2 * H, generator=g).to(dtype)
    a_log, dt = torch.randn(H, generator=g), torch.randn(H, generator=g)
    pos = torch.cat([torch.arange(600), torch.tensor([41]), torch.arange(5, 75),
                     torch.arange(3)]).int()
    state0 = torch.randn(3, H, D, Dv, generator=g) * 0.1
    res = []
    for dev in ("cpu", "cuda"):
        p = proj.to(dev)
        st = state0.clone().to(dev)
        meta = sops.SeqMeta.build(lens, pos.to(dev), dev)
        o = sops.gated_delta_scan(
            p[:, :nqk].unflatten(-1, (G, D)), p[:, nqk : 2 * nqk].unflatten(-1, (G, D)),
            p[:, 2 * nqk : 2 * nqk + nv].unflatten(-1, (H, Dv)),
            p[:, 2 * nqk + nv : 2 * nqk + nv + H], p[:, 2 * nqk + nv + H :],
            a_log.to(dev), dt.to(dev), st, meta)
        res.append((o.cpu(), st.cpu()))
    assert float((res[1][0][:-3] - res[0][0][:-3]).abs().max()) < 1e-4
    assert float((res[1][1] - res[0][1]).abs().max()) < 1e-4
