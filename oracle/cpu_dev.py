"""The CPU device of the MLP step (harness/mlp_step.py): the oracle behind the Matrix method names
(cpu_matrix.CpuMatrix), GEMM on numpy (OpenBLAS).  Test infrastructure, like everything under
oracle/: used by the tests and by the CPU-baseline leg of bench.py only."""
import numpy as np


class CpuDev:
    def __init__(self):
        import cpu_matrix
        import zenu_oracle as zo
        self.M = cpu_matrix.CpuMatrix
        self.sum_to = cpu_matrix.sum_to
        self.F = cpu_matrix      # softmax_backward / cross_entropy / cross_entropy_backward, op by op
        self.zo = zo

    def tick(self, category):
        pass

    def gemm(self, a, b):
        return self.M(np.ascontiguousarray(a.a @ b.a))

    def make_adam(self, params):
        dev = self

        class CpuAdam:
            def __init__(self):
                self.step = 0
                self.m = {k: np.zeros(p.a.size, dtype=p.a.dtype) for k, (p, _) in params.items()}
                self.v = {k: np.zeros(p.a.size, dtype=p.a.dtype) for k, (p, _) in params.items()}

            def update(self, parameters):
                self.step += 1
                for k, (p, g) in parameters.items():
                    f = p.a.dtype.type
                    dev.zo.adam_update(p.a.reshape(-1), np.ascontiguousarray(g.a).reshape(-1), self.m[k], self.v[k],
                                       f(1e-3), f(0.9), f(0.999), f(1e-8), f(self.step))
        return CpuAdam()
