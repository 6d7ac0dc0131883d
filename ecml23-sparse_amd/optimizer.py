"""The optimizer of the reference's training loop: ``SparseAdam`` (sparse/optimizer.py:9-23), a Keras
Adam that also resets its moments where a sparse layer rewires.

The update of every float32 parameter is one pass of ``ffi_adam_step_f32`` in libffi_hip.so (Keras'
update rule, with its defaults ``beta_1=0.9, beta_2=0.999, epsilon=1e-7``); torch holds the tensors.
"""
from __future__ import annotations

import torch

from . import _lib
from .fixed_fan_in_ops import _stream_handle


def adam_step(variable, m, v, gradient, learning_rate, beta_1, beta_2, epsilon, step):
    """One in-place Adam step on contiguous float32 device tensors of equal size; ``step`` counts from 1."""
    for name, t in (("variable", variable), ("m", m), ("v", v), ("gradient", gradient)):
        if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
            raise TypeError(f"{name} must be a contiguous float32 device tensor")
        if t.numel() != variable.numel():
            raise ValueError(f"{name} has {t.numel()} elements, variable has {variable.numel()}")
    with torch.cuda.device(variable.device):
        _lib.check(_lib.lib().ffi_adam_step_f32(variable.data_ptr(), m.data_ptr(), v.data_ptr(), gradient.data_ptr(),
                                                variable.numel(), float(learning_rate), float(beta_1), float(beta_2),
                                                float(epsilon), int(step), _stream_handle(variable.device)))


class SparseAdam:
    """``SparseAdam(params, learning_rate, update_moments=True)``; ``step()`` applies the gradients
    held in ``param.grad`` (Keras' ``apply_gradients``), ``update_sparse(layer)`` rewires a layer and
    clears the moments of the rewired connections (sparse/optimizer.py:14-23)."""

    def __init__(self, params, learning_rate=0.001, beta_1=0.9, beta_2=0.999, epsilon=1e-7, update_moments=True):
        self.params = list(params)
        self.learning_rate = float(learning_rate)
        self.beta_1, self.beta_2, self.epsilon = float(beta_1), float(beta_2), float(epsilon)
        self.update_moments = bool(update_moments)
        self.iterations = 0
        self._momentums = [torch.zeros_like(p.data) for p in self.params]
        self._velocities = [torch.zeros_like(p.data) for p in self.params]

    def zero_grad(self):
        for p in self.params:
            p.grad = None

    @torch.no_grad()
    def step(self):
        self.iterations += 1
        for p, m, v in zip(self.params, self._momentums, self._velocities):
            if p.grad is None:
                continue
            adam_step(p.data, m, v, p.grad.contiguous(), self.learning_rate, self.beta_1, self.beta_2, self.epsilon,
                      self.iterations)

    def _index_of(self, variable):
        for i, p in enumerate(self.params):
            if p is variable:
                return i
        raise KeyError("the variable is not one of this optimizer's parameters")

    def update_sparse(self, layer):
        if self.update_moments:
            i = self._index_of(layer.sparse_weights)
            new_m, new_v = layer.rewire([self._momentums[i], self._velocities[i]])
            self._momentums[i].copy_(new_m)
            self._velocities[i].copy_(new_v)
        else:
            layer.rewire(None)


class SparseOptWrapper(torch.nn.Module):
    """The training loop's model wrapper (sparse/optimizer.py:26-74): ``train_step((x, y))`` runs the base
    model, the loss, the backward pass and the optimizer step, then lets the optimizer rewire every sparse layer
    when ``optimizer.iterations % rewire_interval == 1`` (``rewire_interval <= 0``: never).

    ``compile(optimizer, loss, metrics)`` takes an optimizer with ``zero_grad()``, ``step()``, ``iterations`` and
    ``update_sparse(layer)`` (``SparseAdam``), a loss called as ``loss(y_true, y_pred)`` and metrics with
    ``update_state(y_true, y_pred)`` / ``result()``.  Several optimizers may be given as a list: they are stepped
    together and the first one that has ``update_sparse`` does the rewiring (torch models often keep a stock optimizer
    for their dense layers).
    """

    def __init__(self, rewire_interval: int, base_model: torch.nn.Module):
        super().__init__()
        self.rewire_interval = int(rewire_interval)
        self.base_model = base_model
        self.optimizers = []
        self.loss = None
        self.metrics = []

    def forward(self, *args, **kwargs):
        return self.base_model(*args, **kwargs)

    def compile(self, optimizer, loss, metrics=()):
        self.optimizers = list(optimizer) if isinstance(optimizer, (list, tuple)) else [optimizer]
        if not any(hasattr(o, "update_sparse") for o in self.optimizers):
            raise TypeError("one of the optimizers must have update_sparse(layer)")
        self.loss = loss
        self.metrics = list(metrics)

    @property
    def optimizer(self):
        """The optimizer that rewires (the reference's single optimizer)."""
        return next(o for o in self.optimizers if hasattr(o, "update_sparse"))

    def sparse_layers(self):
        return [m for m in self.base_model.modules() if hasattr(m, "sparse_weights")]

    def train_step(self, data):
        x, y = data
        for o in self.optimizers:
            o.zero_grad()
        y_pred = self.base_model(x)
        loss = self.loss(y, y_pred)
        loss.backward()
        for o in self.optimizers:
            o.step()
        self.handle_sparse_layers()
        results = {"loss": float(loss.detach())}
        with torch.no_grad():
            for m in self.metrics:
                m.update_state(y, y_pred.detach())
                results[getattr(m, "name", type(m).__name__)] = m.result()
        return results

    def handle_sparse_layers(self):
        if self.rewire_interval > 0 and self.optimizer.iterations % self.rewire_interval == 1:
            for layer in self.sparse_layers():
                self.optimizer.update_sparse(layer)


class RewireCallback:
    """Rewires every sparse layer at the start of each epoch but the first (sparse/optimizer.py:77-86)."""

    def __init__(self, model: "SparseOptWrapper"):
        self.model = model

    def on_epoch_begin(self, epoch, logs=None):
        if epoch != 0:
            for layer in self.model.sparse_layers():
                self.model.optimizer.update_sparse(layer)


def backward_sparse_adam(features, lookup, weights, out_grad, nz_words, weight_m, weight_v, bias, bias_m, bias_v,
                         learning_rate, beta_1, beta_2, epsilon, step, transposed=False, grad_is_partial=False,
                         max_density=None, need_feature_grad=True, decide_from_previous=False):
    """Backward pass of the layer and the Adam step on its weights (and bias, unless ``None``) in one call:
    ``weights``, ``bias`` and their moments are updated in place; the weight/bias gradients stay inside the
    library (gradient rows of labels without a non-zero entry of ``out_grad`` are neither written nor read).  Returns ``(feature_grad or None, sparse_kernels_ran)``;
    ``feature_grad`` is formed from the weights as they were on entry."""
    import ctypes

    from .fixed_fan_in_ops import _check_inputs

    batch, num_features, num_units, fan_in = _check_inputs(features, lookup, weights, transposed, out_grad)
    for name, t in (("weights", weights), ("weight_m", weight_m), ("weight_v", weight_v), ("out_grad", out_grad),
                    ("features", features), ("lookup", lookup)):
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous (it is updated or read in place)")
    for name, t in (("weight_m", weight_m), ("weight_v", weight_v)):
        if t.dtype != torch.float32 or t.numel() != weights.numel() or t.device != weights.device:
            raise TypeError(f"{name} must be a float32 tensor with as many elements as weights, on their device")
    if bias is not None:
        for name, t in (("bias", bias), ("bias_m", bias_m), ("bias_v", bias_v)):
            if t is None or t.dtype != torch.float32 or t.numel() != num_units or not t.is_contiguous() or t.device != weights.device:
                raise TypeError(f"{name} must be a contiguous float32 tensor of {num_units} elements on the weights' device")
    taken = ctypes.c_int(-1)
    with torch.cuda.device(features.device):
        feature_grad = torch.empty_like(features) if need_feature_grad else None
        _lib.check(_lib.lib().ffi_backward_sparse_adam_f32(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), out_grad.data_ptr(),
            nz_words.data_ptr() if nz_words is not None else None,
            int(bool(grad_is_partial)) | (2 if decide_from_previous else 0), float(max_density or 0.0),
            feature_grad.data_ptr() if need_feature_grad else None, weight_m.data_ptr(), weight_v.data_ptr(),
            bias.data_ptr() if bias is not None else None, bias_m.data_ptr() if bias is not None else None,
            bias_v.data_ptr() if bias is not None else None,
            float(learning_rate), float(beta_1), float(beta_2), float(epsilon), int(step), ctypes.byref(taken),
            batch, num_features, num_units, fan_in, int(transposed), _stream_handle(features.device)))
    return feature_grad, bool(taken.value)
