"""zenu-optimizer/tests/net_test.rs (sgd_test :107-141, adam_test :143-189, adam_w_test :191-232):
a 2-layer Linear net (2 -> 4 -> 4, no activation) with MSE loss, one or two optimizer steps, compared
with the reference's literal expected parameters (1e-4 / 2e-4).

The forward/backward of the tiny net is restated in numpy here (y = x W^T + b,
zenu-layer/src/layers/linear.rs:19-32; loss = sum((t - y)^2) / t.shape[0],
zenu-autograd/src/loss/mse.rs:6-14) only to produce the gradients; the optimizer updates are the
thing under test: the CPU oracle (pins it) and, on the GPU, the fused HIP kernels."""
import numpy as np
import pytest

import zenu_oracle as zo

F = np.float32


def init_parameters():  # net_test.rs:93-105
    return {
        "linear1.linear.weight": np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 0.07, 0.08], dtype=F).reshape(4, 2),
        "linear1.linear.bias": np.array([0.1, 0.2, 0.3, 0.4], dtype=F),
        "linear2.linear.weight": np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 0.07, 0.08, 0.09, 0.10, 0.11, 0.12, 0.13,
                                           0.14, 0.15, 0.16], dtype=F).reshape(4, 4),
        "linear2.linear.bias": np.array([0.1, 0.2, 0.3, 0.4], dtype=F),
    }


WEIGHTS = ("linear1.linear.weight", "linear2.linear.weight")


def grads(p):
    x = np.array([[0.1, 0.2]], dtype=F)
    t = np.array([0.1, 0.2, 0.3, 0.4], dtype=F)
    h = x @ p["linear1.linear.weight"].T + p["linear1.linear.bias"]
    y = h @ p["linear2.linear.weight"].T + p["linear2.linear.bias"]
    dy = (F(2.0) * (y - t) / F(t.shape[0])).astype(F)          # d/dy of sum((t-y)^2)/4
    dh = dy @ p["linear2.linear.weight"]
    return {"linear1.linear.weight": (dh.T @ x).astype(F), "linear1.linear.bias": dh[0].astype(F),
            "linear2.linear.weight": (dy.T @ h).astype(F), "linear2.linear.bias": dy[0].astype(F)}


SGD_ANS = {
    "linear1.linear.weight": [0.0891, 0.1782, 0.2857, 0.3715, 0.4917, 0.5833, 0.0596, 0.0592],
    "linear1.linear.bias": [-0.0089, 0.0574, 0.2166, 0.2961],
    "linear2.linear.weight": [0.0739, 0.1460, 0.2181, 0.3263, 0.4779, 0.5543, 0.0007, 0.0176, 0.0801, 0.0795, 0.0789,
                              0.0920, 0.1164, 0.1119, 0.1075, 0.1217],
    "linear2.linear.bias": [-0.0742, 0.0525, 0.2339, 0.3095],
}
ADAM_ANS = {
    "linear1.linear.weight": [0.0801, 0.1801, 0.2801, 0.3801, 0.4801, 0.5801, 0.0501, 0.0601],
    "linear1.linear.bias": [0.0801, 0.1801, 0.2801, 0.3801],
    "linear2.linear.weight": [0.0801, 0.1801, 0.2801, 0.3801, 0.4801, 0.5801, 0.0501, 0.0601, 0.0702, 0.0801, 0.0901,
                              0.1001, 0.1101, 0.1201, 0.1301, 0.1401],
    "linear2.linear.bias": [0.0800, 0.1801, 0.2801, 0.3801],
}
ADAMW_ANS = {
    "linear1.linear.weight": [0.0801, 0.1800, 0.2800, 0.3800, 0.4800, 0.5800, 0.0501, 0.0601],
    "linear1.linear.bias": [0.0801, 0.1800, 0.2800, 0.3800],
    "linear2.linear.weight": [0.0801, 0.1800, 0.2800, 0.3800, 0.4800, 0.5800, 0.0501, 0.0601, 0.0702, 0.0801, 0.0901,
                              0.1001, 0.1101, 0.1201, 0.1301, 0.1401],
    "linear2.linear.bias": [0.0800, 0.1800, 0.2801, 0.3800],
}


def check(params, ans, eps):
    for k, v in ans.items():
        got = params[k].reshape(-1).astype(np.float64)
        assert np.max(np.abs(got - np.array(v))) <= eps, (k, got, v)


# ---- CPU oracle ------------------------------------------------------------------------------------

def test_oracle_sgd():
    p = init_parameters()
    g = grads(p)
    for k in p:
        flat = p[k].reshape(-1)
        zo.sgd_update(flat, g[k].reshape(-1).copy(), F(0.9))
    check(p, SGD_ANS, 1e-4)


def test_oracle_adam():
    p = init_parameters()
    for _ in range(2):                                  # two optimizers, each takes its first step
        g = grads(p)
        for k in p:
            m, v = np.zeros(p[k].size, dtype=F), np.zeros(p[k].size, dtype=F)
            zo.adam_update(p[k].reshape(-1), g[k].reshape(-1).copy(), m, v, F(0.01), F(0.9), F(0.999), F(1e-8), F(1))
    check(p, ADAM_ANS, 2e-4)


def test_oracle_adamw():
    p = init_parameters()
    state = {k: (np.zeros(p[k].size, dtype=F), np.zeros(p[k].size, dtype=F)) for k in p}
    for step in (1, 2):                                 # one optimizer, two steps
        g = grads(p)
        for k in p:
            zo.adamw_update(p[k].reshape(-1), g[k].reshape(-1).copy(), *state[k], F(0.01), F(0.9), F(0.999),
                            F(1e-8), F(0.01), k in WEIGHTS, F(step))
    check(p, ADAMW_ANS, 2e-4)


def test_oracle_fused_equals_reference_shaped():
    r = np.random.default_rng(0)
    for dt in (np.float32, np.float64):
        n = 10007
        base = [r.standard_normal(n).astype(dt) * s for s in (0.02, 1e-3, 1e-4)] + [np.abs(r.standard_normal(n).astype(dt)) * 1e-6]
        for adamw in (False, True):
            a = [t.copy() for t in base]
            b = [t.copy() for t in base]
            f = np.dtype(dt).type
            if adamw:
                zo.adamw_update(a[0], a[1], a[2], a[3], f(1e-3), f(0.9), f(0.999), f(1e-8), f(0.01), True, f(10))
            else:
                zo.adam_update(a[0], a[1], a[2], a[3], f(1e-3), f(0.9), f(0.999), f(1e-8), f(10))
            zo.adam_update_fused(b[0], b[1], b[2], b[3], f(1e-3), f(0.9), f(0.999), f(1e-8), f(0.01), True, adamw, f(10))
            for x, y in zip(a, b):
                assert np.array_equal(x, y)


def test_oracle_adam_invariants():
    """closed forms: m = v = 0, t = 1 => |dp| ~ lr, direction -sign(g); lr = 0 => p fixed, m and v move;
    wd = 0 => AdamW == Adam"""
    r = np.random.default_rng(1)
    g = (r.standard_normal(1000) + 3).astype(F) * F(0.01) * np.where(r.random(1000) < 0.5, F(-1), F(1))
    p0 = r.standard_normal(1000).astype(F)
    p, m, v = p0.copy(), np.zeros(1000, dtype=F), np.zeros(1000, dtype=F)
    zo.adam_update(p, g, m, v, F(0.01), F(0.9), F(0.999), F(1e-8), F(1))
    assert np.allclose(p - p0, -0.01 * np.sign(g), rtol=1e-3, atol=1e-6)
    assert np.allclose(m, 0.1 * g, rtol=1e-6) and np.allclose(v, 0.001 * g * g, rtol=1e-5)
    p, m, v = p0.copy(), np.zeros(1000, dtype=F), np.zeros(1000, dtype=F)
    zo.adam_update(p, g, m, v, F(0.0), F(0.9), F(0.999), F(1e-8), F(1))
    assert np.array_equal(p, p0) and np.any(m != 0) and np.any(v != 0)
    a = [p0.copy(), np.zeros(1000, dtype=F), np.zeros(1000, dtype=F)]
    b = [p0.copy(), np.zeros(1000, dtype=F), np.zeros(1000, dtype=F)]
    zo.adam_update(a[0], g, a[1], a[2], F(0.01), F(0.9), F(0.999), F(1e-8), F(3))
    zo.adamw_update(b[0], g, b[1], b[2], F(0.01), F(0.9), F(0.999), F(1e-8), F(0.0), True, F(3))
    assert all(np.array_equal(x, y) for x, y in zip(a, b))


# ---- HIP --------------------------------------------------------------------------------------------

def device_params(hip, p, g):
    return {k: (hip.Matrix.from_numpy(p[k]), hip.Matrix.from_numpy(g[k])) for k in p}


@pytest.mark.gpu
@pytest.mark.parametrize("multi", [True, False])
def test_hip_sgd_net(hip, multi):
    p = init_parameters()
    params = device_params(hip, p, grads(p))
    hip.SGD(0.9).update(params, multi_tensor=multi)
    check({k: v[0].to_numpy() for k, v in params.items()}, SGD_ANS, 1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("multi", [True, False])
def test_hip_adam_net(hip, multi):
    p = init_parameters()
    for _ in range(2):
        params = device_params(hip, p, grads(p))
        hip.Adam(0.01, 0.9, 0.999, 1e-8, params).update(params, multi_tensor=multi)
        p = {k: v[0].to_numpy() for k, v in params.items()}
    check(p, ADAM_ANS, 2e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("multi", [True, False])
def test_hip_adamw_net(hip, multi):
    p = init_parameters()
    params = device_params(hip, p, grads(p))
    opt = hip.AdamW(0.01, 0.9, 0.999, 1e-8, 0.01, params, WEIGHTS)
    for _ in (1, 2):
        g = grads({k: v[0].to_numpy() for k, v in params.items()})
        params = {k: (params[k][0], hip.Matrix.from_numpy(g[k])) for k in params}
        opt.update(params, multi_tensor=multi)
    check({k: v[0].to_numpy() for k, v in params.items()}, ADAMW_ANS, 2e-4)
