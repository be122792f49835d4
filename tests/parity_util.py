"""Shared helpers for the parity tests: seeded inputs, the numpy fp64 policy
evaluation used to cross-check the C oracle, tolerances, and the smoke check.

Tolerance (from the target statement): logits / values / hidden states within
1e-4 relative error of an fp64 evaluation of the same fp32 weights for the fp32
path (2e-2 for bf16 inputs).  "Relative" is taken per tensor against its RMS
magnitude: |got - ref| <= tol * (|ref| + rms(ref)), so entries that cancel to
near zero are judged against the tensor's scale rather than their own.

bf16 inputs: rounding both GEMM operands to 8 significant bits perturbs every
pre-activation by ~0.2 % of its RMS, and three recurrent layers with unit-slope
gates carry that through, so single entries of h3 / state move by up to tens of
percent of the RMS whatever the implementation (numpy_forward_bf16_f64 shows the
same).  The bf16 path is therefore held to (a) 2e-2 in the relative Frobenius
norm against the fp64 oracle and (b) the per-entry metric above, at 2e-3, against
the fp64 evaluation of the SAME bf16-rounded operands.
"""
import numpy as np

HIDDEN, GRU, OBS, OBS_MAP, OBS_TAIL = 256, 768, 843, 792, 51
REC_BYTES, ACTIONS, AV = 996, 43, 44
TOL_FP32 = 1e-4
TOL_BF16 = 2e-2
# a bf16-input result against the fp64 evaluation of the same bf16-rounded operands
TOL_BF16_OPS = 1e-3

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def mix64(seed, stream, index):
    """Counter-based generator shared with the device (csrc/cfp_api.hip mix64)."""
    with np.errstate(over="ignore"):
        idx = np.asarray(index, dtype=np.uint64)
        z = (np.uint64(seed) + np.uint64(stream) * np.uint64(0xD1B54A32D192ED03)
             + (idx + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def unit24(z):
    return (z >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)


def synth_records_host(n, seed, step):
    """Bit-identical host twin of cfp_synth_records: [n][996] uint8."""
    z = mix64(seed, step, np.arange(n * 249, dtype=np.uint64)).reshape(n, 249)
    out = np.empty((n, 249), dtype=np.uint32)
    zm = z[:, :198]
    w = ((zm & np.uint64(0xffff)) % np.uint64(41)).astype(np.uint32)
    w |= (((zm >> np.uint64(16)) & np.uint64(0xffff)) % np.uint64(41)).astype(np.uint32) << 8
    w |= (((zm >> np.uint64(32)) & np.uint64(0xffff)) % np.uint64(41)).astype(np.uint32) << 16
    w |= (((zm >> np.uint64(48)) & np.uint64(0xffff)) % np.uint64(41)).astype(np.uint32) << 24
    out[:, :198] = w
    out[:, 198:] = unit24(z[:, 198:]).view(np.uint32)
    return out.view(np.uint8).reshape(n, REC_BYTES)


def synth_classic_records_host(n, seed, step):
    """Bit-identical host twin of cfp_synth_classic_records: [n][148] uint8."""
    e = np.arange(n, dtype=np.uint64)[:, None] * np.uint64(160)
    out = np.zeros((n, 148), dtype=np.uint8)
    z = mix64(seed, step, e + np.arange(63, dtype=np.uint64)[None, :])
    out[:, :63] = ((z & np.uint64(0xffff)) % np.uint64(17)).astype(np.uint8)
    r = (z >> np.uint64(32)).astype(np.uint64)
    mob = np.where(r % np.uint64(50) == 0, np.uint64(1) + ((r >> np.uint64(8)) % np.uint64(15)),
                   np.uint64(0))
    out[:, 63:126] = mob.astype(np.uint8)
    z = mix64(seed, step, e + np.uint64(64) + np.arange(16, dtype=np.uint64)[None, :])
    out[:, 126:142] = ((z & np.uint64(0xffff)) % np.uint64(10)).astype(np.uint8)
    z = mix64(seed, step, e[:, 0] + np.uint64(80))
    out[:, 142] = (np.uint64(1) + (z & np.uint64(0xffff)) % np.uint64(4)).astype(np.uint8)
    out[:, 143] = ((z >> np.uint64(16)) & np.uint64(1)).astype(np.uint8)
    light = unit24(mix64(seed, step, e[:, 0] + np.uint64(81)))
    out[:, 144:148] = light.view(np.uint8).reshape(n, 4)
    return out


def expand_records(rec):
    """k_expand_obs semantics (craftax_full.cu:10028): bytes -> fp32 features."""
    rec = np.ascontiguousarray(rec).reshape(-1, REC_BYTES)
    x = np.empty((rec.shape[0], OBS), dtype=np.float32)
    x[:, :OBS_MAP] = rec[:, :OBS_MAP].astype(np.float32)
    x[:, OBS_MAP:] = np.ascontiguousarray(rec[:, OBS_MAP:]).view(np.float32)
    return x


def random_params(layers, seed, scale=1.0, obs=None, actions=None):
    """Xavier-uniform-ish random weights in the flat arena layout."""
    OBS_, ACTIONS_ = (obs or OBS), (actions or ACTIONS)
    rng = np.random.default_rng(seed)
    def u(shape, bound):
        return rng.uniform(-bound, bound, size=shape).astype(np.float32)
    parts = [
        u((OBS_ * HIDDEN,), scale * np.sqrt(6.0 / (OBS_ + HIDDEN))),
        u((HIDDEN,), 1.0 / np.sqrt(OBS_)),
        u((layers * GRU * HIDDEN,), scale * np.sqrt(6.0 / (HIDDEN + GRU))),
        u((ACTIONS_ * HIDDEN,), scale * np.sqrt(6.0 / (HIDDEN + ACTIONS_))),
        u((ACTIONS_,), 1.0 / np.sqrt(HIDDEN)),
        u((HIDDEN,), scale * np.sqrt(6.0 / (HIDDEN + 1))),
        u((1,), 1.0 / np.sqrt(HIDDEN)),
    ]
    return np.concatenate(parts)


def split_params(params, layers, obs=None, actions=None):
    OBS_, ACTIONS_ = (obs or OBS), (actions or ACTIONS)
    o = {}
    off = 0
    for name, shape in (("W_enc", (OBS_, HIDDEN)), ("b_enc", (HIDDEN,)),
                        ("W_gru", (layers, GRU, HIDDEN)), ("W_a", (ACTIONS_, HIDDEN)),
                        ("b_a", (ACTIONS_,)), ("W_v", (HIDDEN,)), ("b_v", (1,))):
        cnt = int(np.prod(shape))
        o[name] = np.asarray(params[off:off + cnt]).reshape(shape)
        off += cnt
    assert off == len(params)
    return o


def sigmoid64(z):
    return 1.0 / (1.0 + np.exp(-z))


def numpy_forward_f64(params, layers, x, state, terminals, obs=None, actions=None):
    """Independent fp64 evaluation with library matmuls (A.2 of the forward spec:
    craftax_full.cu:9778-9854).  x [n][843], state [L][n][256] -> dict of fp64
    arrays; state is not modified."""
    w = {k: v.astype(np.float64)
         for k, v in split_params(params, layers, obs, actions).items()}
    h = x.astype(np.float64) @ w["W_enc"] + w["b_enc"]
    out = {"h_enc": h.copy()}
    new_state = np.empty((layers,) + h.shape, dtype=np.float64)
    r_state = np.empty_like(new_state)
    dz = (np.asarray(terminals) != 0)[:, None]
    for l in range(layers):
        st = np.where(dz, 0.0, state[l].astype(np.float64))
        r_state[l] = st
        z = h @ w["W_gru"][l].T
        zh, zg, zp = z[:, :HIDDEN], z[:, HIDDEN:2 * HIDDEN], z[:, 2 * HIDDEN:]
        gh = np.where(zh >= 0.0, zh + 0.5, sigmoid64(zh))
        o = st + sigmoid64(zg) * (gh - st)
        p = sigmoid64(zp)
        h = p * o + (1.0 - p) * h
        new_state[l] = o
    out["h3"] = h
    out["state"] = new_state
    out["r_state"] = r_state
    out["logits"] = h @ w["W_a"].T + w["b_a"]
    out["values"] = h @ w["W_v"] + w["b_v"][0]
    return out


def bf16_round(a):
    """Round to the nearest bf16 (ties to even); result as fp64."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + np.uint64(0x7FFF) + ((u >> np.uint64(16)) & np.uint64(1))) & np.uint64(0xFFFF0000)
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a)).astype(np.float64)


def numpy_forward_bf16_f64(params, layers, x, state, terminals, obs=None, actions=None,
                           quantize_encoder=True):
    """fp64 evaluation of the bf16-input forward: both operands of the encoder, gate
    and head GEMMs are rounded to bf16 (the activations from their fp32 value),
    products and sums are exact/fp64, everything else as numpy_forward_f64."""
    w = {k: v.astype(np.float64)
         for k, v in split_params(params, layers, obs, actions).items()}
    q = bf16_round
    f32 = lambda a: a.astype(np.float32)
    if quantize_encoder:
        h = q(x) @ q(w["W_enc"]) + w["b_enc"]
    else:
        h = x.astype(np.float64) @ w["W_enc"] + w["b_enc"]
    out = {"h_enc": h.copy()}
    new_state = np.empty((layers,) + h.shape, dtype=np.float64)
    dz = (np.asarray(terminals) != 0)[:, None]
    for l in range(layers):
        st = np.where(dz, 0.0, state[l].astype(np.float64))
        z = q(f32(h)) @ q(w["W_gru"][l]).T
        zh, zg, zp = z[:, :HIDDEN], z[:, HIDDEN:2 * HIDDEN], z[:, 2 * HIDDEN:]
        gh = np.where(zh >= 0.0, zh + 0.5, sigmoid64(zh))
        o = st + sigmoid64(zg) * (gh - st)
        p = sigmoid64(zp)
        h = p * o + (1.0 - p) * h
        new_state[l] = o
    out["h3"] = h
    out["state"] = new_state
    out["logits"] = q(f32(h)) @ q(w["W_a"]).T + w["b_a"]
    out["values"] = q(f32(h)) @ q(w["W_v"]) + w["b_v"][0]
    return out


def numpy_ppo_backward_f64(params, layers, feats, r_state, r_act, r_logprob, adv, ret, r_done,
                           seg_len, clip=0.2, vf=0.5, ent=0.01, mode=0, map_rows_exact=False):
    """The PPO update's gradients (recompute from the stored state, reverse sweep with the
    carry cut at segment ends and blocked at terminal steps; k_head_bwd_win,
    k_mingru_bwd_win and the GEMMs of cu_train_backward, craftax_full.cu:9635-9689,
    9560-9620, 13230-13330) in fp64 with library matmuls, over all envs at once.
    feats [T][n][843], r_state [T][L][n][256].
    mode 0: exact operands.  mode 1: both operands of every matrix product rounded to bf16
    (activations and gradients from their fp32 value); with map_rows_exact the 768 leading
    map bytes multiply the unrounded encoder gradient (an exact three-term split of it, what
    the update does with the split kernels off).  mode 2: also what the bf16 window storage rounds -- the gate
    pre-activations and layer inputs as the sweep reads them, the gate gradients and the
    highway term as written, the outputs of the dh GEMMs.
    Returns (gradient vector, [pg, v, ent] sums)."""
    T, n = r_act.shape
    H = HIDDEN
    w = {k: v.astype(np.float64) for k, v in split_params(params, layers).items()}
    f32 = lambda a: np.asarray(a, dtype=np.float64).astype(np.float32)
    q = (lambda a: bf16_round(f32(a))) if mode else (lambda a: np.asarray(a, dtype=np.float64))
    qs = (lambda a: bf16_round(f32(a))) if mode == 2 else (lambda a: np.asarray(a, dtype=np.float64))
    We, Wg, Wa, Wv = q(w["W_enc"]), q(w["W_gru"]), q(w["W_a"]), q(w["W_v"])
    a64 = adv.astype(np.float32).astype(np.float64)
    mean = a64.sum() / (n * T)
    var = max((a64 * a64).sum() / (n * T) - mean * mean, 0.0)
    inv_std = 1.0 / (np.sqrt(var) + 1e-8)
    inv_batch = 1.0 / (T * n)
    clip, vf, ent = (float(np.float32(c)) for c in (clip, vf, ent))
    g = {k: np.zeros_like(v) for k, v in w.items()}
    loss3 = np.zeros(3)
    carry = np.zeros((layers, n, H))
    rows = np.arange(n)
    for t in range(T - 1, -1, -1):
        # ---- recompute
        x = [q(feats[t]) @ We + w["b_enc"]]
        zs, outs = [], []
        for l in range(layers):
            z = q(x[l]) @ Wg[l].T
            zh, zg, zp = z[:, :H], z[:, H:2 * H], z[:, 2 * H:]
            st = r_state[t, l].astype(np.float64)
            gh = np.where(zh >= 0.0, zh + 0.5, sigmoid64(zh))
            o = st + sigmoid64(zg) * (gh - st)
            pm = sigmoid64(zp)
            x.append(pm * o + (1.0 - pm) * x[l])
            zs.append((zh, zg, zp))
        h3q = q(x[layers])
        lg = h3q @ Wa.T + w["b_a"]
        val = h3q @ Wv + w["b_v"][0]
        # ---- head
        lse = np.log(np.exp(lg - lg.max(1, keepdims=True)).sum(1, keepdims=True)) + lg.max(1, keepdims=True)
        logp = lg - lse
        pi = np.exp(logp)
        act = r_act[t]
        ratio = np.exp(logp[rows, act] - r_logprob[t].astype(np.float64))
        A = (a64[t] - mean) * inv_std
        u1 = ratio * A
        u2 = np.clip(ratio, 1.0 - clip, 1.0 + clip) * A
        dlogp = np.where(u1 <= u2, -A * ratio, 0.0)
        Hent = -(pi * logp).sum(1)
        dret = val - ret[t].astype(np.float64)
        loss3 += [-np.minimum(u1, u2).sum(), (0.5 * dret * dret).sum(), Hent.sum()]
        onehot = np.zeros_like(pi); onehot[rows, act] = 1.0
        dlog = (dlogp[:, None] * (onehot - pi) + ent * pi * (logp + Hent[:, None])) * inv_batch
        dv = inv_batch * vf * dret
        g["b_a"] += dlog.sum(0); g["b_v"] += dv.sum()
        g["W_a"] += q(dlog).T @ h3q
        g["W_v"] += q(dv) @ h3q
        dh = qs(q(dlog) @ Wa + q(dv)[:, None] * Wv[None, :])
        # ---- reverse layers
        cut = (t == T - 1) or ((t + 1) % seg_len == 0)
        passes = (r_done[t] == 0).astype(np.float64)[:, None]
        dhx = np.zeros((n, H))
        for l in range(layers - 1, -1, -1):
            if cut:
                carry[l] = 0.0
            zh, zg, zp = (qs(z) for z in zs[l])
            st = r_state[t, l].astype(np.float64)
            top = dh + dhx
            sg, pm = sigmoid64(zg), sigmoid64(zp)
            gh = np.where(zh >= 0.0, zh + 0.5, sigmoid64(zh))
            dgh = np.where(zh >= 0.0, 1.0, sigmoid64(zh) * (1.0 - sigmoid64(zh)))
            o = st + sg * (gh - st)
            dout = top * pm + passes * carry[l]
            dzp = qs(top * (o - qs(x[l])) * pm * (1.0 - pm))
            dhx = qs(top * (1.0 - pm))
            carry[l] = dout * (1.0 - sg)
            dzg = qs(dout * (gh - st) * sg * (1.0 - sg))
            dzh = qs(dout * sg * dgh)
            dpre = q(np.concatenate([dzh, dzg, dzp], axis=1))
            g["W_gru"][l] += dpre.T @ q(x[l])
            dh = dpre @ Wg[l]
            if l > 0:
                dh = qs(dh)
        dh = qs(dh + dhx)
        g["b_enc"] += dh.sum(0)
        ft = feats[t].astype(np.float64)
        g["W_enc"][:768] += ft[:, :768].T @ (dh if map_rows_exact else q(dh))
        g["W_enc"][768:] += q(ft[:, 768:]).T @ q(dh)
    flat = np.concatenate([g[k].ravel() for k in ("W_enc", "b_enc", "W_gru", "W_a", "b_a", "W_v", "b_v")])
    return flat, loss3


def fro_err(got, ref):
    """Relative Frobenius error ||got - ref|| / ||ref||."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.sqrt(np.sum((got - ref) ** 2)) / (np.sqrt(np.sum(ref * ref)) + 1e-30))


def rel_err(got, ref):
    """max over entries of |got-ref| / (|ref| + rms(ref))."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = np.sqrt(np.mean(ref * ref)) + 1e-30
    return float(np.max(np.abs(got - ref) / (np.abs(ref) + rms)))


def strict_rel_err(got, ref):
    """max of |got-ref| / |ref| over the entries with |ref| >= rms(ref): the plain relative
    error where it is well defined (entries that are not the result of a cancellation)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    big = (np.abs(ref) >= np.sqrt(np.mean(ref * ref))) & (ref != 0)
    if not big.any():
        return 0.0
    return float(np.max(np.abs(got - ref)[big] / np.abs(ref)[big]))


def assert_close(got, ref, tol, what):
    """Two bounds: |got-ref| <= tol * (|ref| + rms(ref)) for every entry, and the plain
    |got-ref| <= tol * |ref| for every entry at least as large as the rms."""
    e = rel_err(got, ref)
    assert np.all(np.isfinite(np.asarray(got))), f"{what}: non-finite values"
    assert e <= tol, f"{what}: relative error {e:.3e} exceeds {tol:.1e}"
    es = strict_rel_err(got, ref)
    assert es <= tol, f"{what}: plain relative error {es:.3e} of the large entries exceeds {tol:.1e}"
    return e


def smoke_forward(pkg):
    """One small fused forward on cuda:0 against the CPU oracle."""
    import torch
    import oracle_bind
    n, layers = 64, 3
    params = random_params(layers, 11)
    pol = pkg.Policy(n, layers, seed=1)
    pol.set_params(params)
    rec_h = synth_records_host(n, 5, 0)
    rng = np.random.default_rng(3)
    state_h = (0.5 * rng.standard_normal((layers, n, HIDDEN))).astype(np.float32)
    term_h = (rng.random(n) < 0.25).astype(np.float32)
    rec = torch.from_numpy(rec_h).cuda()
    state = torch.from_numpy(state_h.copy()).cuda()
    term = torch.from_numpy(term_h).cuda()
    av = pol.forward(rec, term, state)
    torch.cuda.synchronize()
    ref = oracle_bind.forward_f64(params, layers, expand_records(rec_h), state_h, term_h)
    av_h = av.cpu().numpy()
    assert_close(av_h[:, :ACTIONS], ref["logits"], TOL_FP32, "smoke logits")
    assert_close(av_h[:, ACTIONS], ref["values"], TOL_FP32, "smoke values")
    assert_close(state.cpu().numpy(), ref["state"], TOL_FP32, "smoke state")
    pol.close()


def smoke_env(pkg):
    """64 envs generated and stepped 20 times on cuda:0 against the compiled reference env
    (oracle/_ref), every state field after every step; skipped when the checker is not built."""
    import torch
    import env_bind as eb
    try:
        ref = eb.Ref()
    except FileNotFoundError:
        print("smoke: oracle/_ref/libcfref.so is not built, env check skipped")
        return
    n, seed = 64, 5
    ref.init(n, seed)
    env = pkg.Env(n)
    env.init(seed)
    assert not eb.diff_fields(ref.export(), env.export_states(eb.STATE_DTYPE)), "smoke: generated worlds differ"
    for t in range(20):
        act = ref.next_actions()
        final, rew, term, keys = ref.step(act)
        env.step(None)
        bad = eb.diff_fields(final, env.export_states(eb.STATE_DTYPE))
        assert not bad, f"smoke: env step {t}: fields {bad[:4]} differ from the reference"
        assert np.array_equal(rew.view(np.uint32), env.rewards.cpu().numpy().view(np.uint32))
        env.reset()
    env.close()
