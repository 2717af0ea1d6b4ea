"""Optimizers behind the reference's `Optimizer::update` surface, one fused launch per step.

  SGD    zenu-optimizer/src/sgd.rs:6-31
  Adam   zenu-optimizer/src/adam.rs:9-89
  AdamW  zenu-optimizer/src/adamw.rs:9-101

`parameters` is what `Parameters::parameters()` yields in the reference
(zenu-layer/src/lib.rs:27-41): a mapping name -> (param Matrix, grad Matrix or None); for AdamW
`weights` names the keys of `Parameters::weights()` (only those get weight decay).  Parameters
must be default-stride (they are whole tensors in the reference too).
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import check
from .matrix import Matrix, get_stream, _dt


def _flat(m):
    if not m.is_default_stride_strict():
        raise ValueError("optimizer tensors must be default stride")
    return m.as_ptr(), m.num_elm()


class SGD:
    def __init__(self, learning_rate):
        self.learning_rate = learning_rate

    def update(self, parameters, multi_tensor=True):
        items = [(d, g) for _, (d, g) in parameters.items() if g is not None]
        if not items:
            return
        dtype = items[0][0].dtype
        if multi_tensor and all(d.dtype == dtype for d, _ in items):
            n = len(items)
            P, G = (C.c_void_p * n)(), (C.c_void_p * n)()
            sizes = (C.c_int64 * n)()
            for i, (d, g) in enumerate(items):
                P[i], sizes[i] = _flat(d)
                G[i] = _flat(g)[0]
            check(_lib.lib().zenu_hip_sgd_step_multi(_dt(dtype), n, P, G, sizes, float(self.learning_rate),
                                                     get_stream()), "sgd_step_multi")
            return
        for data, grad in items:
            p, n = _flat(data)
            g, _ = _flat(grad)
            check(_lib.lib().zenu_hip_sgd_step(_dt(data.dtype), p, g, n, float(self.learning_rate),
                                               get_stream()), "sgd_step")


class _AdamBase:
    def __init__(self, learning_rate, beta1, beta2, epsilon, parameters):
        self.learning_rate, self.beta1, self.beta2, self.epsilon = learning_rate, beta1, beta2, epsilon
        self.step = 0
        # zeros_like per parameter (adam.rs:62-88)
        self.m = {k: Matrix.zeros(p.shape, p.dtype) for k, (p, _) in parameters.items()}
        self.v = {k: Matrix.zeros(p.shape, p.dtype) for k, (p, _) in parameters.items()}
        self._schedule = None

    def use_schedule(self, n_steps, dtype=np.float32):
        """Take the step-dependent scalars of the next `n_steps` updates from a table in device memory
        whose cursor every update advances, so that an `update` recorded into a HIP graph is the next
        step on every replay (no counterpart in the reference, which never records graphs)."""
        self.drop_schedule()
        h = C.c_void_p()
        check(_lib.lib().zenu_hip_adam_schedule_create(C.byref(h), _dt(dtype), float(self.beta1), float(self.beta2),
                                                       self.step + 1, int(n_steps), get_stream()), "adam_schedule_create")
        self._schedule = h
        self._schedule_dtype = np.dtype(dtype)

    def drop_schedule(self):
        if self._schedule is not None:
            check(_lib.lib().zenu_hip_adam_schedule_destroy(self._schedule, get_stream()), "adam_schedule_destroy")
            self._schedule = None

    def schedule_state(self):
        """(next step, steps left in the table, updates refused because the table had run out)"""
        a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
        check(_lib.lib().zenu_hip_adam_schedule_query(self._schedule, C.byref(a), C.byref(b), C.byref(c), get_stream()),
              "adam_schedule_query")
        return a.value, b.value, c.value

    def __del__(self):
        try:
            self.drop_schedule()
        except Exception:
            pass

    def _update(self, parameters, weight_decay, weight_keys, multi):
        self.step += 1
        items = [(k, d, g) for k, (d, g) in parameters.items() if g is not None]
        if not items:
            return
        dtype = items[0][1].dtype
        if multi and all(d.dtype == dtype for _, d, _ in items):
            n = len(items)
            arr = lambda: (C.c_void_p * n)()
            P, G, M, V = arr(), arr(), arr(), arr()
            sizes = (C.c_int64 * n)()
            decay = (C.c_int32 * n)()
            for i, (k, d, g) in enumerate(items):
                P[i], sizes[i] = _flat(d)
                G[i] = _flat(g)[0]
                M[i] = _flat(self.m[k])[0]
                V[i] = _flat(self.v[k])[0]
                decay[i] = 1 if (weight_keys is not None and k in weight_keys) else 0
            if self._schedule is not None:
                if np.dtype(dtype) != self._schedule_dtype:
                    raise ValueError("the schedule was made for another dtype")
                check(_lib.lib().zenu_hip_adam_step_multi_scheduled(
                    _dt(dtype), n, P, G, M, V, sizes, float(self.learning_rate), float(self.epsilon),
                    float(weight_decay), decay, self._schedule, get_stream()), "adam_step_multi_scheduled")
                return
            check(_lib.lib().zenu_hip_adam_step_multi(
                _dt(dtype), n, P, G, M, V, sizes, float(self.learning_rate), float(self.beta1),
                float(self.beta2), float(self.epsilon), float(weight_decay), decay, float(self.step),
                get_stream()), "adam_step_multi")
            return
        if self._schedule is not None:
            raise ValueError("a scheduled update takes the multi-tensor path: one dtype, multi_tensor=True")
        for k, d, g in items:
            p, n = _flat(d)
            decay = 1 if (weight_keys is not None and k in weight_keys) else 0
            check(_lib.lib().zenu_hip_adamw_step(
                _dt(d.dtype), p, _flat(g)[0], _flat(self.m[k])[0], _flat(self.v[k])[0], n,
                float(self.learning_rate), float(self.beta1), float(self.beta2), float(self.epsilon),
                float(weight_decay), decay, float(self.step), get_stream()), "adamw_step")


class Adam(_AdamBase):
    def update(self, parameters, multi_tensor=True):
        self._update(parameters, 0.0, None, multi_tensor)


class AdamW(_AdamBase):
    def __init__(self, learning_rate, beta1, beta2, epsilon, weight_decay, parameters, weights):
        super().__init__(learning_rate, beta1, beta2, epsilon, parameters)
        self.weight_decay = weight_decay
        self.weight_keys = set(weights)

    def update(self, parameters, multi_tensor=True):
        self._update(parameters, self.weight_decay, self.weight_keys, multi_tensor)
