"""BASELINE config[4]: one training step of the MNIST-shaped MLP (Linear 784-512-ReLU-512-ReLU-10,
softmax cross-entropy, backward, one Adam step), replayed as the sequence of zenu-matrix ops that
ZeNu's autograd issues, written once against the Matrix API and run on either device (CpuMatrix =
oracle, zenu_amd.Matrix = HIP).  Used by tests/test_mlp_step.py and bench.py.

Op sequence followed (reference file:line):
  Linear::call            transpose(W) materialised, matmul, + bias     zenu-layer/src/layers/linear.rs:23-32,
                                                                        zenu-autograd/src/functions/transpose.rs:26-33
  relu / backward mask                                                  zenu-autograd/src/activation/relu.rs:24-47
  softmax_assign          x - max_axis(1,keep), exp, sum(1,keep), /=    zenu-matrix/src/operation/softmax.rs:10-25
  cross_entropy           log, * target, sum_to([]), / (-N)             zenu-autograd/src/loss/cross_entropy.rs:12-23
  backward of div / sum_to / mul / log / softmax / add / matmul / transpose
                                                                        zenu-autograd/src/functions/{div,sum_to,mul,log,add,
                                                                        matmul,transpose}.rs, loss/softmax.rs:33-40
  set_grad on a broadcast operand = sum_to                              zenu-autograd/src/lib.rs:466-486
  Adam::update                                                          zenu-optimizer/src/adam.rs:19-59

With fused=True the same step uses the fused entry points (bias add + ReLU, softmax cross-entropy
forward and backward, ReLU backward, the two backward calls also producing the bias gradients): 30
launches instead of 62 on the HIP device.  On the CPU
device those names are the op-by-op chains, so both settings compute the same thing there.

GEMM stays on the library path (`dev.gemm`): numpy/OpenBLAS for the CPU leg, rocBLAS for the HIP
leg.  `dev.tick(category)` lets the caller attribute time to gemm / elementwise / reduction / copy /
update.
"""
import numpy as np

LAYERS = [(784, 512), (512, 512), (512, 10)]
BATCH = 256


def make_inputs(seed=4, dtype=np.float32):
    """x ~ U[0,1) [256,784], one-hot labels [256,10], W ~ N(0,1)/sqrt(fan_in), b = 0
    (zenu-layer/src/layers/linear.rs:56-68)"""
    r = np.random.default_rng(seed)
    x = r.random((BATCH, 784)).astype(dtype)
    labels = r.integers(0, 10, BATCH)
    t = np.zeros((BATCH, 10), dtype=dtype)
    t[np.arange(BATCH), labels] = 1
    params = {}
    for i, (fin, fout) in enumerate(LAYERS, 1):
        params[f"linear{i}.weight"] = (r.standard_normal((fout, fin)) / np.sqrt(fin)).astype(dtype)
        params[f"linear{i}.bias"] = np.zeros(fout, dtype=dtype)
    return x, t, params


class MlpStep:
    """dev needs: M (matrix class), sum_to(src, target), gemm(a, b) -> a @ b (contiguous operands),
    tick(category), make_adam(params) -> optimizer with update(params)"""

    def __init__(self, dev, x, t, params, fused=False):
        self.dev = dev
        self.fused = fused
        M = dev.M
        self.x, self.t = M.from_numpy(x), M.from_numpy(t)
        self.p = {k: M.from_numpy(v) for k, v in params.items()}
        self.opt = dev.make_adam({k: (v, None) for k, v in self.p.items()})
        self.dtype = x.dtype
        # 0-d constants live on the device for the whole run (Variable::from(-n), the seed gradient)
        self.neg_n = M.from_vec([-float(BATCH)], [], x.dtype)
        self.one = M.from_vec([1.0], [], x.dtype)

    def _linear_fwd(self, i, x):
        tick = self.dev.tick
        W, b = self.p[f"linear{i}.weight"], self.p[f"linear{i}.bias"]
        Wt = W.transpose().to_default_stride(); tick("copy")          # transpose(W): a materialised copy
        z = self.dev.gemm(x, Wt); tick("gemm")
        a = z + b; tick("elementwise")                                 # broadcast add, one launch
        return Wt, a

    def _linear_relu_fwd(self, i, x):
        """fused: (Wt, pre-activation, activation) with one launch for `+ bias` and relu"""
        tick = self.dev.tick
        W, b = self.p[f"linear{i}.weight"], self.p[f"linear{i}.bias"]
        Wt = W.transpose().to_default_stride(); tick("copy")
        z = self.dev.gemm(x, Wt); tick("gemm")
        a, h = z.alloc_like(), z.alloc_like()
        h.bias_add_relu(z, b, 0.0, pre=a); tick("elementwise")
        return Wt, a, h

    def step(self):
        return self._step_fused() if self.fused else self._step_ops()

    def _step_fused(self):
        dev, M, tick = self.dev, self.dev.M, self.dev.tick
        dt = self.dtype
        Wt1, a1, h1 = self._linear_relu_fwd(1, self.x)
        Wt2, a2, h2 = self._linear_relu_fwd(2, h1)
        Wt3, logits = self._linear_fwd(3, h2)
        loss, s = dev.F.cross_entropy(logits, self.t); tick("reduction")
        # each bias gradient comes out of the launch that produces the gradient it sums (no zero fill:
        # it is overwritten)
        gb = M.alloc([LAYERS[2][1]], dt)
        g = dev.F.cross_entropy_backward_bias_grad(s, self.t, gb, self.one); tick("reduction")
        grads = {}
        acts = [(self.x, Wt1, a1), (h1, Wt2, a2), (h2, Wt3, None)]
        for i in (3, 2, 1):
            inp, Wt, _ = acts[i - 1]
            grads[f"linear{i}.bias"] = gb
            inpT = inp.transpose().to_default_stride(); tick("copy")
            gWt = dev.gemm(inpT, g); tick("gemm")
            grads[f"linear{i}.weight"] = gWt.transpose().to_default_stride(); tick("copy")
            if i > 1:
                WtT = Wt.transpose().to_default_stride(); tick("copy")
                g_h = dev.gemm(g, WtT); tick("gemm")
                g = g_h.alloc_like(); gb = M.alloc([LAYERS[i - 2][1]], dt)
                g.relu_backward_bias_grad(gb, g_h, acts[i - 2][2], 0.0); tick("elementwise")
        self.opt.update({k: (self.p[k], grads[k]) for k in self.p}); tick("update")
        return loss, grads

    def _step_ops(self):
        dev, M, tick = self.dev, self.dev.M, self.dev.tick
        dt = self.dtype
        # ---- forward ---------------------------------------------------------------------------
        Wt1, a1 = self._linear_fwd(1, self.x)
        h1 = a1.alloc_like(); h1.relu(a1, 0.0); tick("elementwise")
        Wt2, a2 = self._linear_fwd(2, h1)
        h2 = a2.alloc_like(); h2.relu(a2, 0.0); tick("elementwise")
        Wt3, logits = self._linear_fwd(3, h2)
        # softmax_assign
        mx = logits.max_axis(1, True); tick("reduction")
        diff = logits - mx; tick("elementwise")
        e = diff.exp(); tick("elementwise")
        sm = e.sum(1, True); tick("reduction")
        e /= sm; tick("elementwise")
        s = e.alloc_like(); s.copy_from(e); tick("copy")
        lg = s.log(); tick("elementwise")
        yl = self.t * lg; tick("elementwise")
        total = M.zeros([], dt); dev.sum_to(yl, total); tick("reduction")
        neg_n = self.neg_n
        loss = total / neg_n; tick("elementwise")
        # ---- backward ----------------------------------------------------------------------------
        g_total = self.one / neg_n; tick("elementwise")                      # div backward, x side
        g_yl = M.zeros([BATCH, 10], dt); g_yl += g_total; tick("elementwise")   # broadcast(g, shape)
        g_lg = self.t * g_yl; tick("elementwise")                       # mul backward, y side
        g_s = g_lg / s; tick("elementwise")                             # log backward
        gx = s * g_s; tick("elementwise")                               # softmax backward
        sum_gx = gx.sum(1, True); tick("reduction")
        tmp = s * sum_gx; tick("elementwise")
        g_logits = gx - tmp; tick("elementwise")
        grads = {}
        g = g_logits
        acts = [(self.x, Wt1, a1), (h1, Wt2, a2), (h2, Wt3, None)]
        for i in (3, 2, 1):
            inp, Wt, _ = acts[i - 1]
            gb = M.zeros([LAYERS[i - 1][1]], dt); dev.sum_to(g, gb); tick("reduction")   # bias grad
            grads[f"linear{i}.bias"] = gb
            inpT = inp.transpose().to_default_stride(); tick("copy")
            gWt = dev.gemm(inpT, g); tick("gemm")                        # dW^T = X^T dY
            grads[f"linear{i}.weight"] = gWt.transpose().to_default_stride(); tick("copy")
            if i > 1:
                WtT = Wt.transpose().to_default_stride(); tick("copy")
                g_h = dev.gemm(g, WtT); tick("gemm")                     # dX = dY W
                a_prev = acts[i - 2][2]
                mask = a_prev.alloc_like(); mask.relu_backward_mask(a_prev, 0.0); tick("elementwise")
                g = g_h * mask; tick("elementwise")
        # ---- Adam ----------------------------------------------------------------------------------
        self.opt.update({k: (self.p[k], grads[k]) for k in self.p}); tick("update")
        return loss, grads
