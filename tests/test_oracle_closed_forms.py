"""Pins the parts of the CPU checker that the seeded SAC loop does not exercise (it uses ReLU/identity layers, all-true masks,
external noise) by what the mathematics fixes: closed forms, finite differences, brute force on tiny inputs, invariants."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import Mlp, capi


def test_activations_and_derivatives(oracle):
    lib = oracle.lib
    xs = np.linspace(-4, 4, 161).astype(np.float32)
    closed = {
        "identity": lambda x: x, "relu": lambda x: np.maximum(x, 0), "tanh": np.tanh, "sigmoid": lambda x: 1 / (1 + np.exp(-x)),
        # the reference's tanh-GELU uses a = FRAC_2_SQRTPI * SQRT1_2 * 0.5 = sqrt(2/pi)/2 (nn/activation_functions.h:33-36), half the
        # textbook constant; parity is with the reference
        "gelu": lambda x: 0.5 * x * (1 + np.tanh(0.5 * np.sqrt(2 / np.pi) * (x + 0.044715 * x ** 3))),
        "fast_tanh": lambda x: (lambda c: c * (27 + c * c) / (27 + 9 * c * c))(np.clip(x, -3, 3)),
    }
    for name, f in closed.items():
        got = np.array([lib.rlt_oracle_activation(float(x), capi.ACT[name]) for x in xs])
        assert np.allclose(got, f(xs.astype(np.float64)), rtol=2e-6, atol=2e-6), name
        d = np.array([lib.rlt_oracle_d_activation(float(x), capi.ACT[name]) for x in xs])
        h = 1e-4
        fd = (f(xs.astype(np.float64) + h) - f(xs.astype(np.float64) - h)) / (2 * h)
        if name == "fast_tanh":     # the reference DEFINES this derivative as 1 - fast_tanh(x)^2 (nn/activation_functions.h:76-79), not the slope of the rational
            assert np.allclose(d, 1 - f(xs.astype(np.float64)) ** 2, atol=2e-6)
            continue
        keep = np.abs(xs) > 1e-3 if name == "relu" else np.ones_like(xs, bool)
        assert np.allclose(d[keep], fd[keep], rtol=1e-4, atol=1e-4), name


@pytest.mark.parametrize("acts", [("tanh", "identity"), ("sigmoid", "tanh"), ("gelu", "identity"), ("relu", "sigmoid")])
def test_mlp_gradients_by_finite_differences(oracle, acts):
    """loss = sum(dy * y): the analytic d/dW, d/db, d/dx of the checker's backward against central differences of its forward
    (fp64 accumulation so the difference quotient is clean)."""
    oracle.lib.rlt_oracle_set_f64_accumulate(1)
    try:
        rng = np.random.default_rng(0)
        B, dims = 3, [4, 5, 5, 2]
        params = helpers.random_params(rng, dims, bias_scale=0.5)
        x = rng.standard_normal((B, 4)).astype(np.float32)
        dy = rng.standard_normal((B, 2)).astype(np.float32)

        def loss(p, xin):
            net = Mlp(oracle, dims, p, B, acts[0], acts[1])
            xd, yd = oracle.array(xin), oracle.zeros((B, 2))
            oracle.call("mlp_evaluate", net.layers, net.n, xd.ptr, 4, yd.ptr, 2, B, None, 0)
            return float((yd.numpy().astype(np.float64) * dy).sum())

        net = Mlp(oracle, dims, params, B, acts[0], acts[1])
        xd, dyd, dxd = oracle.array(x), oracle.array(dy), oracle.zeros((B, 4))
        oracle.call("mlp_zero_gradient", net.layers, net.n)
        oracle.call("mlp_forward", net.layers, net.n, xd.ptr, 4, B)
        oracle.call("mlp_backward", net.layers, net.n, xd.ptr, 4, dyd.ptr, 2, dxd.ptr, 4, B, 1, None, 0)
        grads, dx = net.grads.numpy(), dxd.numpy()
        h = 1e-2
        for i in rng.choice(params.size, 25, replace=False):
            pp, pm = params.copy(), params.copy()
            pp[i] += h; pm[i] -= h
            fd = (loss(pp, x) - loss(pm, x)) / (pp[i] - pm[i])
            assert abs(fd - grads[i]) <= 2e-3 * max(1.0, abs(fd)), (i, fd, grads[i])
        for b in range(B):
            for j in range(4):
                xp, xm = x.copy(), x.copy()
                xp[b, j] += h; xm[b, j] -= h
                fd = (loss(params, xp) - loss(params, xm)) / (xp[b, j] - xm[b, j])
                assert abs(fd - dx[b, j]) <= 2e-3 * max(1.0, abs(fd))
    finally:
        oracle.lib.rlt_oracle_set_f64_accumulate(0)


def test_dense_forward_is_affine_map_plus_activation(oracle):
    rng = np.random.default_rng(1)
    B, I, O = 7, 5, 3
    W, b = rng.standard_normal((O, I)).astype(np.float32), rng.standard_normal(O).astype(np.float32)
    x = rng.standard_normal((B, I + 2)).astype(np.float32)      # leading dimension wider than the layer input
    net = Mlp(oracle, [I, O], np.concatenate([W.ravel(), b]), B, out_act="tanh")
    xd, yd = oracle.array(x), oracle.zeros((B, O + 1))
    oracle.call("dense_evaluate", C.pointer(net.layers[0]), xd.ptr, I + 2, yd.ptr, O + 1, B)
    want = np.tanh(x[:, :I].astype(np.float64) @ W.T.astype(np.float64) + b)
    assert np.allclose(yd.numpy()[:, :O], want, atol=1e-6) and np.all(yd.numpy()[:, O] == 0)


def test_adam_first_step_closed_form_and_epsilon_sqrt_clamp(oracle):
    """With m = v = 0 and age = 1 the bias corrections cancel the (1-beta) factors: delta = alpha * g / (|g| + eps), and where
    g^2 < eps_sqrt the denominator is sqrt(eps_sqrt) + eps instead."""
    g = np.array([1.0, -2.5, 1e-3, -1e-5, 0.0], np.float32)
    p0 = np.zeros(5, np.float32)          # zero so that the step itself is what is stored
    for eps in (1e-7, 1e-8):
        arrs = [oracle.array(a) for a in (p0, g, np.zeros(5, np.float32), np.zeros(5, np.float32))]
        age = oracle.array(np.array([1], np.uint32))
        t = (capi.AdamTensor * 1)(capi.AdamTensor(arrs[0].ptr, arrs[1].ptr, arrs[2].ptr, arrs[3].ptr, None, 5, 0))
        par = capi.adam_parameters(epsilon=eps)
        oracle.call("adam_step", t, 1, C.byref(par), age.ptr, 0.0, None)
        g64 = g.astype(np.float64)
        denom = np.sqrt(np.maximum(g64 ** 2, eps)) + eps
        assert np.allclose(p0 - arrs[0].numpy(), 1e-3 * g64 / denom, rtol=1e-4, atol=1e-9)
        assert age.numpy()[0] == 2
        assert np.allclose(arrs[2].numpy(), 0.1 * g, rtol=1e-6) and np.allclose(arrs[3].numpy(), 0.001 * g * g, rtol=5e-5)   # 1 - 0.999f is 1.3e-5 off 0.001


def test_adam_matches_textbook_recursion(oracle):
    """Five steps against the textbook Adam recursion in float64 (Kingma & Ba, eps added outside the square root)."""
    rng = np.random.default_rng(2)
    n = 64
    p = rng.standard_normal(n); m = np.zeros(n); v = np.zeros(n)
    arrs = [oracle.array(a.astype(np.float32)) for a in (p, np.zeros(n), m, v)]
    age = oracle.array(np.array([1], np.uint32))
    t = (capi.AdamTensor * 1)(capi.AdamTensor(arrs[0].ptr, arrs[1].ptr, arrs[2].ptr, arrs[3].ptr, None, n, 0))
    par = capi.adam_parameters(epsilon=1e-8)
    for step in range(1, 6):
        g = rng.standard_normal(n).astype(np.float32)
        arrs[1].upload(g)
        oracle.call("adam_step", t, 1, C.byref(par), age.ptr, 0.0, None)
        m = 0.9 * m + 0.1 * g; v = 0.999 * v + 0.001 * g.astype(np.float64) ** 2
        p = p - 1e-3 * (m / (1 - 0.9 ** step)) / (np.sqrt(v / (1 - 0.999 ** step)) + 1e-8)
    assert np.allclose(arrs[0].numpy(), p, rtol=2e-5, atol=2e-6)


def test_polyak_and_mse(oracle):
    rng = np.random.default_rng(3)
    s, t = rng.standard_normal(100).astype(np.float32), rng.standard_normal(100).astype(np.float32)
    sd, td = oracle.array(s), oracle.array(t)
    oracle.call("polyak_update", sd.ptr, td.ptr, 100, 0.995, 0)
    assert np.allclose(td.numpy(), 0.995 * t + 0.005 * s, rtol=1e-6, atol=1e-7)
    td2 = oracle.array(t)
    oracle.call("polyak_update", sd.ptr, td2.ptr, 100, 0.999, 1)
    assert np.allclose(td2.numpy(), 0.999 * t + 0.001 * s * s, rtol=1e-6, atol=1e-7)
    a, b = rng.standard_normal((10, 3)).astype(np.float32), rng.standard_normal((10, 3)).astype(np.float32)
    ad, bd, dd, ld = oracle.array(a), oracle.array(b), oracle.zeros((10, 3)), oracle.zeros((1,))
    oracle.call("mse_gradient", ad.ptr, 3, bd.ptr, 3, dd.ptr, 3, 10, 3, 0.5, None)
    oracle.call("mse_evaluate", ad.ptr, 3, bd.ptr, 3, 10, 3, 0.5, ld.ptr)
    assert np.allclose(dd.numpy(), (a - b) * 2 / 30 * 0.5, rtol=1e-6)
    assert np.isclose(ld.numpy()[0], ((a - b) ** 2).mean() * 0.5, rtol=1e-6)


def test_sample_and_squash_closed_form_invariants_and_finite_differences(oracle):
    rng = np.random.default_rng(4)
    B, D = 6, 2
    inp = np.concatenate([0.5 * rng.standard_normal((B, D)), rng.uniform(-1.5, 0.0, (B, D))], 1).astype(np.float32)
    inp[0, D] = 5.0; inp[1, D + 1] = -30.0       # outside the clamp range [-20, 2]
    noise = rng.standard_normal((B, D)).astype(np.float32)
    p = capi.SasParameters(-20.0, 2.0, 1e-6, -float(D))
    log_alpha = np.float32(np.log(0.3))

    def forward(x, nz):
        xd, nd = oracle.array(x), (oracle.array(nz) if nz is not None else None)
        act, pre, lp = oracle.zeros((B, D)), oracle.zeros((B, D)), oracle.zeros((B,))
        oracle.call("sas_forward", C.byref(p), xd.ptr, 2 * D, nd.ptr if nd else None, D, act.ptr, D, pre.ptr, D, lp.ptr, B, D)
        return act.numpy(), pre.numpy(), lp.numpy()

    act, pre, lp = forward(inp, noise)
    ls = np.clip(inp[:, D:].astype(np.float64), -20, 2)
    sample = inp[:, :D] + noise * np.exp(ls)
    # 1 - a^2 + 1e-6 cancels catastrophically for saturated actions, so that term is formed in fp32 from the fp32 action, as any
    # fp32 implementation must; the Gaussian part is checked in float64
    squash = np.log((np.float32(1) - act * act + np.float32(1e-6)).astype(np.float32)).astype(np.float64)
    # z is taken from the fp32 sample: with log_std clamped at -20 the noise term is below one ulp of the mean and z rounds to 0
    z = (pre.astype(np.float64) - inp[:, :D]) / np.exp(ls)
    want_lp = (-0.5 * np.log(2 * np.pi) - ls - 0.5 * z ** 2 - squash).sum(1)
    assert np.allclose(act, np.tanh(sample), atol=1e-6) and np.all(np.abs(act) <= 1) and np.allclose(pre, sample, atol=1e-5)
    assert np.allclose(lp, want_lp, rtol=1e-5, atol=1e-5)
    act0, _, lp0 = forward(inp, None)              # evaluation mode: the mean is the sample, z = 0
    assert np.allclose(act0, np.tanh(inp[:, :D]), atol=1e-6)
    # backward against central differences of  L = sum_b [ g_b . a_b + alpha/B * logp_b ]  wrt the layer input
    g = rng.standard_normal((B, D)).astype(np.float32)
    alpha = float(np.exp(log_alpha))

    def L(x):
        a, _, l = forward(x, noise)
        return float((a.astype(np.float64) * g).sum() + alpha / B * l.astype(np.float64).sum())

    xd, nd, ad, pd, gd = (oracle.array(v) for v in (inp, noise, act, pre, g))
    din = oracle.zeros((B, 2 * D)); la = oracle.array(np.array([log_alpha])); dla = oracle.array(np.array([1.5], np.float32))
    oracle.call("sas_backward", C.byref(p), xd.ptr, 2 * D, nd.ptr, D, ad.ptr, D, pd.ptr, D, gd.ptr, D, din.ptr, 2 * D, la.ptr, dla.ptr, B, D)
    din = din.numpy()
    h = 1e-3
    # rows 0 and 1 sit outside the clamp (saturated tanh / sigma = e^-20): there the reference's analytic formula, which drops the
    # 1e-6 inside the log, is not the slope of the fp32 forward; they are checked for the gating only
    for b in range(2, B):
        for j in range(2 * D):
            xp, xm = inp.copy(), inp.copy()
            xp[b, j] += h; xm[b, j] -= h
            fd = (L(xp) - L(xm)) / (float(xp[b, j]) - float(xm[b, j]))
            assert abs(fd - din[b, j]) <= 5e-3 * max(1.0, abs(fd)), (b, j, fd, din[b, j])
    assert din[0, D] == 0 and din[1, D + 1] == 0                                   # gated by the clamp
    # d_log_alpha is INCREMENTED by mean_b alpha * (-logp_b - target_entropy)
    assert np.isclose(dla.numpy()[0], 1.5 + np.mean(alpha * (-lp.astype(np.float64) + D)), rtol=1e-5)


def test_target_values_min_q_and_masks_brute_force(oracle):
    rng = np.random.default_rng(5)
    B = 9
    q1, q2, r, lp = (rng.standard_normal(B).astype(np.float32) for _ in range(4))
    term = np.array([0, 1, 0, 0, 1, 0, 0, 0, 1], np.uint8)
    arr = {k: oracle.array(v) for k, v in dict(q1=q1, q2=q2, r=r, lp=lp, term=term).items()}
    la, y = oracle.array(np.array([np.log(0.2)], np.float32)), oracle.zeros((B,))
    oracle.call("sac_target_action_values", arr["q1"].ptr, arr["q2"].ptr, arr["r"].ptr, arr["term"].ptr, arr["lp"].ptr, la.ptr, 0.99, 0, y.ptr, B)
    want = [r[i] + (0.0 if term[i] else 0.99 * (min(q1[i], q2[i]) - 0.2 * lp[i])) for i in range(B)]
    assert np.allclose(y.numpy(), want, rtol=1e-6, atol=1e-6)
    d1, d2 = rng.standard_normal((B, 5)).astype(np.float32), rng.standard_normal((B, 5)).astype(np.float32)
    out = oracle.zeros((B, 2))
    oracle.call("sac_min_value_d_output", arr["q1"].ptr, arr["q2"].ptr, oracle.array(d1).ptr, oracle.array(d2).ptr, 5, 5, 2, out.ptr, 2, B)
    d1d, d2d = oracle.array(d1), oracle.array(d2)
    oracle.call("sac_min_value_d_output", arr["q1"].ptr, arr["q2"].ptr, d1d.ptr, d2d.ptr, 5, 5, 2, out.ptr, 2, B)
    for i in range(B):
        assert np.array_equal(out.numpy()[i], (d1 if q1[i] < q2[i] else d2)[i, 3:])
    mask = np.array([1, 0, 1, 1, 0, 0, 1, 0, 1], np.uint8)
    src, dst = rng.standard_normal((B, 2)).astype(np.float32), rng.standard_normal((B, 2)).astype(np.float32)
    md, sd, dd = oracle.array(mask), oracle.array(src), oracle.array(dst)
    oracle.call("mask_copy", sd.ptr, 2, dd.ptr, 2, md.ptr, 1, B, 2)          # inverted: rows with mask == 0 are copied
    assert np.array_equal(dd.numpy(), np.where(mask[:, None] == 0, src, dst))
    gd = oracle.array(src)
    oracle.call("mask_zero", gd.ptr, 2, md.ptr, 1, B, 2)
    assert np.array_equal(gd.numpy(), np.where(mask[:, None] == 0, 0, src))


def test_gae_brute_force_with_terminations_and_truncations(oracle):
    """A_t = sum_k (gamma*lambda)^k delta_{t+k} within an episode segment, delta = r + gamma*V' - V; a terminated step bootstraps
    with 0, a truncated-but-not-terminated step contributes delta = 0 and cuts the sum (rl/algorithms/ppo/operations_generic.h:60-95)."""
    rng = np.random.default_rng(6)
    n_envs, steps, gamma, lam = 3, 12, 0.9, 0.8
    rows = (steps + 1) * n_envs
    r, v = rng.standard_normal(rows), rng.standard_normal(rows)
    term = np.zeros(rows); trunc = np.zeros(rows)
    term[[4 * n_envs + 0, 7 * n_envs + 1]] = 1; trunc[[4 * n_envs + 0, 7 * n_envs + 1, 9 * n_envs + 2, 2 * n_envs + 1]] = 1
    cols = [oracle.array(c.astype(np.float32)) for c in (r, term, trunc, v)]
    adv, tv = oracle.zeros((rows,)), oracle.zeros((rows,))
    oracle.call("ppo_gae", cols[0].ptr, cols[1].ptr, cols[2].ptr, cols[3].ptr, adv.ptr, tv.ptr, 1, n_envs, steps, gamma, lam, 0)
    adv, tv = adv.numpy(), tv.numpy()
    for env in range(n_envs):
        for t in range(steps):
            total, k = 0.0, 0
            while t + k < steps:
                pos = (t + k) * n_envs + env
                v_next = 0.0 if term[pos] else v[pos + n_envs]
                delta = r[pos] + gamma * v_next - v[pos]
                if trunc[pos] and not term[pos]:
                    delta = 0.0
                total += (gamma * lam) ** k * delta
                if trunc[pos]:
                    break
                k += 1
            pos = t * n_envs + env
            assert abs(adv[pos] - total) <= 1e-5 * max(1, abs(total)), (env, t)
            assert abs(tv[pos] - (total + v[pos])) <= 1e-5 * max(1, abs(total + v[pos]))


def test_pendulum_matches_gymnasium_equations(oracle):
    """Pendulum-v1 (Gymnasium classic_control/pendulum.py): thdot' = clip(thdot + (3g/2l sin th + 3/(ml^2) u) dt, +-8),
    th' = th + thdot' dt, cost = angle_normalize(th)^2 + 0.1 thdot^2 + 0.001 u^2 from the pre-step state; the reference does not
    clip u in the reward."""
    rng = np.random.default_rng(7)
    N = 200
    th, thd = rng.uniform(-10, 10, N), rng.uniform(-8, 8, N)
    a = rng.uniform(-1.5, 1.5, N)
    s = oracle.array(np.stack([th, thd], 1).astype(np.float32)); ad = oracle.array(a.astype(np.float32))
    o, no, r = oracle.zeros((N, 3)), oracle.zeros((N, 3)), oracle.zeros((N,))
    p = capi.pendulum_parameters()
    oracle.call("pendulum_step", C.byref(p), s.ptr, ad.ptr, o.ptr, no.ptr, r.ptr, N)
    th32, thd32, a32 = th.astype(np.float32).astype(np.float64), thd.astype(np.float32).astype(np.float64), a.astype(np.float32).astype(np.float64)
    u = 2 * np.clip(a32, -1, 1)
    nthd = np.clip(thd32 + (15 * np.sin(th32) + 3 * u) * 0.05, -8, 8)
    nth = th32 + nthd * 0.05
    norm = ((th32 + np.pi) % (2 * np.pi)) - np.pi
    cost = norm ** 2 + 0.1 * thd32 ** 2 + 0.001 * (2 * a32) ** 2
    assert np.allclose(s.numpy(), np.stack([nth, nthd], 1), rtol=1e-5, atol=1e-5)
    assert np.allclose(r.numpy(), -cost, rtol=1e-5, atol=1e-4)
    assert np.allclose(o.numpy(), np.stack([np.cos(th32), np.sin(th32), thd32], 1), atol=1e-6)
    assert np.allclose(no.numpy(), np.stack([np.cos(nth), np.sin(nth), nthd], 1), atol=1e-5)


def test_gather_deterministic_mode_and_ring_index_brute_force(oracle):
    """DETERMINISTIC gather takes offset = sample number (tests/src/rl/cuda/rl.cu:201-228). Ring index once full:
    (position + MAX_EPISODE_LENGTH + offset) % CAPACITY, checked against an explicit list model of the ring."""
    cap, n_add = 12, 31
    rb = helpers.ReplayOnBackend(oracle, 1, cap)
    ring = [None] * cap
    pos = 0
    for i in range(n_add):
        obs, nobs = np.full((1, 3), i, np.float32), np.full((1, 3), i + 0.5, np.float32)
        args = [oracle.array(v) for v in (obs, np.array([[-i]], np.float32), np.array([i * 10], np.float32), nobs, np.array([i % 5 == 0], np.uint8), np.array([i % 7 == 0], np.uint8))]
        oracle.call("replay_add", C.byref(rb.c), *[a.ptr for a in args])
        ring[pos] = i; pos = (pos + 1) % cap
    assert rb.position.numpy()[0] == pos and rb.full.numpy()[0] == 1
    B, max_ep = 8, 5
    oab, rew, term = oracle.zeros((2, B, 4)), oracle.zeros((B,)), oracle.zeros((B,), np.uint8)
    oracle.call("gather_batch", C.byref(rb.c), None, None, 1, max_ep, B, oab.ptr, rew.ptr, term.ptr, None, None, None, None)
    for s in range(B):
        i = ring[(pos + max_ep + s) % cap]
        assert np.all(oab.numpy()[0, s, :3] == i) and oab.numpy()[0, s, 3] == -i and rew.numpy()[s] == i * 10
        assert np.all(oab.numpy()[1, s, :3] == i + 0.5) and oab.numpy()[1, s, 3] == 0 and term.numpy()[s] == (i % 5 == 0)


def test_evaluation_with_a_standardize_layer_is_the_plain_one_with_folded_statistics(oracle):
    """(x - m) * p in front of W x + b is W' x + b' with W' = W diag(p), b' = b - W' m: the checker's standardized evaluation against its plain
    evaluation of the folded network (short horizon: the fold changes the rounding), and identity statistics against the plain one exactly."""
    rng = np.random.default_rng(11)
    dims = [3, 24, 24, 1]
    params = helpers.random_params(rng, dims)
    n = 12
    ini = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
    mean, precision = rng.normal(0, 0.5, 3).astype(np.float32), rng.uniform(0.3, 3, 3).astype(np.float32)
    plain = helpers.evaluate_on_backend(oracle, dims, params, "tanh", "identity", 1, ini, 10)
    same = helpers.evaluate_on_backend(oracle, dims, params, "tanh", "identity", 1, ini, 10, (np.zeros(3), np.ones(3)))
    assert np.array_equal(plain[0], same[0]) and np.array_equal(plain[2], same[2])
    got = helpers.evaluate_on_backend(oracle, dims, params, "tanh", "identity", 1, ini, 10, (mean, precision))
    folded = helpers.fold_standardize_into_first_layer(dims, params, mean, precision)
    want = helpers.evaluate_on_backend(oracle, dims, folded, "tanh", "identity", 1, ini, 10)
    assert helpers.rel_err(got[0], want[0]) <= 1e-4 and helpers.rel_err(got[0], plain[0]) > 1e-2
