"""BASELINE config[4]: the MLP training step on the HIP library against the same step on the CPU
oracle (same op sequence, same inputs; GEMM on each side's library).

Bars: quantities that do not pass through a GEMM-dependent chain would be bit-exact; everything
here sits downstream of GEMMs computed by two different libraries (OpenBLAS vs rocBLAS, different
summation order), so loss, gradients and updated parameters are compared at 1e-4 relative to the
tensor's largest magnitude."""
import numpy as np
import pytest

import cpu_dev
from harness import hip_dev, mlp_step


def rel(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) / max(np.max(np.abs(b)), 1e-30))


def test_cpu_step_matches_plain_numpy():
    """pins the op sequence itself: the oracle-run step equals a direct numpy forward/backward"""
    x, t, params = mlp_step.make_inputs()
    cpu = mlp_step.MlpStep(cpu_dev.CpuDev(), x, t, params)
    loss, grads = cpu.step()
    W1, b1, W2, b2, W3, b3 = (params[f"linear{i}.{n}"].astype(np.float64) for i in (1, 2, 3) for n in ("weight", "bias"))
    xd, td = x.astype(np.float64), t.astype(np.float64)
    a1 = xd @ W1.T + b1; h1 = np.maximum(a1, 0)
    a2 = h1 @ W2.T + b2; h2 = np.maximum(a2, 0)
    z = h2 @ W3.T + b3
    s = np.exp(z - z.max(1, keepdims=True)); s /= s.sum(1, keepdims=True)
    ref_loss = -(td * np.log(s)).sum() / x.shape[0]
    gz = (s - td) / x.shape[0]
    assert abs(float(loss.to_numpy()) - ref_loss) / ref_loss < 1e-5
    assert rel(grads["linear3.weight"].to_numpy(), gz.T @ h2) < 1e-4
    assert rel(grads["linear3.bias"].to_numpy(), gz.sum(0)) < 1e-4
    g2 = (gz @ W3) * (a2 > 0)
    assert rel(grads["linear2.weight"].to_numpy(), g2.T @ h1) < 1e-4
    g1 = (g2 @ W2) * (a1 > 0)
    assert rel(grads["linear1.weight"].to_numpy(), g1.T @ xd) < 1e-4
    assert rel(grads["linear1.bias"].to_numpy(), g1.sum(0)) < 1e-4


def test_cpu_fused_spelling_is_the_same_chain():
    """on the CPU device the fused names are the op-by-op chains: identical bits"""
    x, t, params = mlp_step.make_inputs()
    a = mlp_step.MlpStep(cpu_dev.CpuDev(), x, t, params)
    b = mlp_step.MlpStep(cpu_dev.CpuDev(), x, t, params, fused=True)
    la, ga = a.step()
    lb, gb = b.step()
    assert np.array_equal(la.to_numpy(), lb.to_numpy())
    for k in ga:
        assert np.array_equal(ga[k].to_numpy(), gb[k].to_numpy()), k
        assert np.array_equal(a.p[k].to_numpy(), b.p[k].to_numpy()), k


@pytest.mark.gpu
def test_hip_fused_step_matches_hip_step(hip):
    """fused entry points against the op sequence on the same device and the same GEMMs: they differ
    only in summation order (softmax denominators over 10 classes, the loss), far below 1e-5"""
    x, t, params = mlp_step.make_inputs()
    dev = hip_dev.HipDev(hip)
    a = mlp_step.MlpStep(dev, x, t, params)
    b = mlp_step.MlpStep(dev, x, t, params, fused=True)
    for step in range(3):
        for k in a.p:                      # same starting point each step
            b.p[k].copy_from(a.p[k]); b.opt.m[k].copy_from(a.opt.m[k]); b.opt.v[k].copy_from(a.opt.v[k])
        la, ga = a.step()
        lb, gb = b.step()
        assert abs(float(la.to_numpy()) - float(lb.to_numpy())) <= 1e-5 * abs(float(la.to_numpy()))
        for k in ga:
            assert rel(gb[k].to_numpy(), ga[k].to_numpy()) < 1e-5, (step, k)


def write_inputs(path, x, t, params):
    """raw f32 in the order harness/native/mlp_step_bench.cpp reads"""
    with open(path, "wb") as f:
        for a in [x, t] + [params[f"linear{i}.{n}"] for i in (1, 2, 3) for n in ("weight", "bias")]:
            f.write(np.ascontiguousarray(a, dtype=np.float32).tobytes())


@pytest.mark.gpu
def test_compiled_host_step_matches_python_host(hip, tmp_path):
    """the same step issued from C++ (include/zenu_hip.hpp + rocBLAS): same kernels, same GEMM library, so
    the losses of the first steps agree to rounding noise of the launch-order-independent kernels"""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "harness", "native", "bin", "mlp_step_bench")
    if not os.path.exists(exe):
        pytest.skip("harness/native/bin/mlp_step_bench is not built (run __graft_entry__.build())")
    x, t, params = mlp_step.make_inputs()
    write_inputs(tmp_path / "inputs.bin", x, t, params)
    out = subprocess.run([exe, "--inputs", str(tmp_path / "inputs.bin"), "--dump-loss", "3", "--steps", "2", "--warmup", "0"],
                         capture_output=True, text=True, timeout=100)
    print(out.stdout, flush=True)
    assert out.returncode == 0, out.stdout + out.stderr
    got = {(l.split()[0], int(l.split()[2])): float(l.split()[3]) for l in out.stdout.splitlines() if " loss " in l}
    dev = hip_dev.HipDev(hip)
    for fused in (False, True):
        st = mlp_step.MlpStep(dev, x, t, params, fused=fused)
        for step in (1, 2, 3):
            loss, _ = st.step()
            ref = float(loss.to_numpy())
            assert abs(got[("fused" if fused else "ops", step)] - ref) <= 1e-6 * abs(ref), (fused, step)
    # the variant whose GEMMs read transposed views instead of copies: other GEMM kernels, so 1e-4
    for step in (1, 2, 3):
        assert abs(got[("lean", step)] - got[("fused", step)]) <= 1e-4 * abs(got[("fused", step)]), step


@pytest.mark.gpu
def test_hip_step_matches_cpu_step(hip):
    import zenu_oracle as zo
    x, t, params = mlp_step.make_inputs()
    cpu = mlp_step.MlpStep(cpu_dev.CpuDev(), x, t, params)
    dev = hip_dev.HipDev(hip)
    gpu = mlp_step.MlpStep(dev, x, t, params)
    losses = []
    for step in range(1, 4):
        print(f"[c4] step {step}", flush=True)
        # both legs start the step from the GPU's state, so GEMM rounding does not accumulate
        p0 = {k: v.to_numpy() for k, v in gpu.p.items()}
        m0 = {k: v.to_numpy().reshape(-1) for k, v in gpu.opt.m.items()}
        v0 = {k: v.to_numpy().reshape(-1) for k, v in gpu.opt.v.items()}
        for k in cpu.p:
            cpu.p[k].a[...] = p0[k]
        closs, cgrads = cpu.step()
        gloss, ggrads = gpu.step()
        losses.append(float(gloss.to_numpy()))
        # loss and gradients sit downstream of GEMMs from two libraries: 1e-4
        assert abs(losses[-1] - float(closs.to_numpy())) / abs(float(closs.to_numpy())) < 1e-4
        for k in cgrads:
            assert rel(ggrads[k].to_numpy(), cgrads[k].to_numpy()) < 1e-4, (step, k)
        # the fused Adam update, fed the GPU's own gradients, is bit-exact against the oracle
        # (Adam's g / (|g| + eps) amplifies GEMM rounding on near-zero gradients, so the
        # cross-library parameters are not compared directly)
        f = np.float32
        for k in p0:
            pe = p0[k].reshape(-1).copy()
            zo.adam_update(pe, ggrads[k].to_numpy().reshape(-1), m0[k], v0[k], f(1e-3), f(0.9), f(0.999), f(1e-8), f(step))
            assert np.array_equal(pe, gpu.p[k].to_numpy().reshape(-1)), (step, k)
            assert np.array_equal(m0[k], gpu.opt.m[k].to_numpy().reshape(-1)), (step, k)
            assert np.array_equal(v0[k], gpu.opt.v[k].to_numpy().reshape(-1)), (step, k)
    assert losses[2] < losses[0]          # it trains
