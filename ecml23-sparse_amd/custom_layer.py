"""The caller of the fixed-fan-in ops: a torch module shaped like the reference's layer.

Mirrors ``StratifiedRewireLayerV2`` (sparse/custom_layer.py:6-50) on top of ``RewireLayerBase``
(sparse/layer.py:106-249): flat variables of ``connections`` entries, viewed as
``[units, connections // units]`` at call time; column ids drawn uniformly with replacement; the
call is the transposed op followed by a bias add (here one fused kernel); rewiring replaces the
sources of the selected connections in place and clears the matching entries of optimizer state.
Everything on the call path runs in libffi_hip.so; torch holds the variables.
"""
from __future__ import annotations

import math

import torch

from . import fixed_fan_in_ops as ops


class RewireSelector:
    """Decides which connections a rewiring step replaces (sparse/layer.py:30-44): ``select(weight_values)``
    returns a boolean tensor, true where a connection shall be rewired.  A selector may also offer
    ``threshold_tensor(weight_values)`` (rewire everything strictly below a magnitude): the layer then selects,
    redraws and clears optimizer state in one library call instead of torch index operations."""

    def select(self, weight_values: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError()

    def build(self, weight_values: torch.Tensor):
        pass


class FixedMagnitudeSelector(RewireSelector):
    """Rewire all weights below a fixed magnitude (sparse/layer.py:45-57)."""

    def __init__(self, threshold: float):
        self.threshold = float(threshold)

    def select(self, weight_values: torch.Tensor) -> torch.Tensor:
        return weight_values.abs() < self.threshold

    def threshold_tensor(self, weight_values: torch.Tensor) -> torch.Tensor:
        """The magnitude below which connections are rewired, as a device tensor ``[1]``."""
        return torch.full((1,), self.threshold, dtype=torch.float32, device=weight_values.device)


class FixedFractionSelector(RewireSelector):
    """Rewire a fixed fraction of the connections, those of lowest magnitude (sparse/layer.py:60-84).

    As in the reference the threshold is the ``round(fraction * n)``-th smallest magnitude and the
    comparison is strict, so the connection that defines the threshold (and its ties) stays.
    """

    def __init__(self, fraction: float):
        if not 0.0 <= fraction <= 1.0:
            raise ValueError(f"Received an invalid value {fraction} for `fraction`, expected 0.0 <=  fraction <= 1.0")
        self.fraction = float(fraction)

    def select(self, weight_values: torch.Tensor) -> torch.Tensor:
        flat = weight_values.reshape(-1).abs()
        num_selected = int(round(self.fraction * flat.numel()))
        if num_selected <= 0:
            return torch.zeros_like(flat, dtype=torch.bool)
        threshold = torch.kthvalue(flat, num_selected).values
        return flat < threshold

    def threshold_tensor(self, weight_values: torch.Tensor) -> torch.Tensor:
        """The same threshold by the library's radix select (device tensor ``[1]``; 0 selects nothing)."""
        flat = weight_values.detach().reshape(-1).contiguous()
        return ops.select_threshold(flat, int(round(self.fraction * flat.numel())))


class StratifiedRewireLayerV2(torch.nn.Module):
    """Fixed-fan-in sparse layer: ``units`` outputs, each fed by ``connections // units`` inputs."""

    def __init__(self, units: int, input_dim: int, *, connections: int | None = None, sparsity: float | None = None,
                 use_bias: bool = True, rewire_selector=None, arrange: bool = True, device="cuda",
                 generator: torch.Generator | None = None):
        super().__init__()
        if int(units) != units or units < 0:
            raise ValueError(f"Received an invalid value for `units`, expected a positive integer, got {units}.")
        if sparsity is not None and connections is not None:
            raise ValueError("The `sparsity` and `connections` arguments are mutually exclusive")
        if sparsity is None and connections is None:
            raise ValueError("one of `sparsity` and `connections` is needed")
        if sparsity is not None and not 0.0 <= sparsity <= 1.0:
            raise ValueError(f"Received an invalid value {sparsity} for `sparsity`, expected 0.0 <=  sparsity <= 1.0")
        self.units = int(units)
        self.input_dim = int(input_dim)
        # sparse/layer.py:173-177
        self.connections = int(connections) if connections is not None else int((self.units * self.input_dim) * (1.0 - sparsity))
        if self.connections < self.units or self.connections % self.units != 0:
            raise ValueError("connections must be a positive multiple of units (the op views them as [units, fan_in])")
        self.use_bias = bool(use_bias)
        self.rewire_selector = rewire_selector if rewire_selector is not None else FixedFractionSelector(0.01)
        self._generator = generator
        # seeds of the rewiring draws: a base taken from the generator (or torch's global seed) plus a call counter
        self._rewire_seed = int(generator.initial_seed() if generator is not None else torch.initial_seed()) * 1000003
        self._rewire_count = 0
        # one weight per connection, Keras' default 'glorot_uniform' on a rank-1 shape: fan_in = fan_out = connections
        limit = math.sqrt(6.0 / (2.0 * self.connections))
        w = (torch.rand(self.connections, device=device, generator=generator) * 2.0 - 1.0) * limit
        self.kernel_weights = torch.nn.Parameter(w)
        # sources drawn uniformly, with replacement (sparse/custom_layer.py:12-15); the reference stores
        # them as uint32, the same bits as the int32 kept here
        self.register_buffer("kernel_indices", self._random_sources(self.connections, device))
        self.bias = torch.nn.Parameter(torch.zeros(self.units, device=device)) if self.use_bias else None
        # keep every label's connections in the order the kernels read fastest (see arrange_connections);
        # no counterpart in the reference, where the order inside a row is arbitrary as well
        self.arrange = bool(arrange) and torch.device(device).type == "cuda"
        if self.arrange:
            self.arrange_connections()

    @torch.no_grad()
    def arrange_connections(self, other_vars=None):
        """Reorders each label's connections (indices, weights and ``other_vars`` together) in place."""
        others = [] if other_vars is None else [o.view(-1, self.fan_in) for o in other_vars]
        ops.arrange_connections(self.kernel_indices.view(-1, self.fan_in), self.kernel_weights.data.view(-1, self.fan_in), *others)

    @property
    def fan_in(self) -> int:
        return self.connections // self.units

    def _random_sources(self, count: int, device) -> torch.Tensor:
        return torch.randint(0, self.input_dim, (count,), device=device, generator=self._generator, dtype=torch.int64).to(torch.int32)

    # sparse/custom_layer.py:45-50 followed by the bias add of sparse/layer.py:245-247
    def _sparse_matmul(self, inputs: torch.Tensor) -> torch.Tensor:
        indices = self.kernel_indices.view(-1, self.fan_in)
        weights = self.kernel_weights.view(-1, self.fan_in)
        tp_in = inputs.t().contiguous()
        return ops.fan_in_sparse_matmul_tp(tp_in, indices, weights)

    @property
    def sparse_weights(self):
        """The variable an optimizer keeps moments for (sparse/layer.py:160-162)."""
        return self.kernel_weights

    def forward(self, inputs: torch.Tensor) -> torch.Tensor:
        if inputs.dim() != 2 or inputs.shape[1] != self.input_dim:
            raise ValueError(f"inputs must have shape [batch, {self.input_dim}], got {tuple(inputs.shape)}")
        if inputs.dtype != torch.float32:
            inputs = inputs.float()
        if not self.use_bias:
            return self._sparse_matmul(inputs)
        # same result as _sparse_matmul(inputs) + bias; the [B,N] entry point transposes inside the library
        indices = self.kernel_indices.view(-1, self.fan_in)
        weights = self.kernel_weights.view(-1, self.fan_in)
        return ops.fan_in_sparse_matmul_bias(inputs, indices, weights, self.bias)

    def forward_loss(self, inputs: torch.Tensor, y_true, loss, want_scores: bool = False):
        """``loss(y_true, self(inputs))`` with the loss gradient formed inside the forward kernel:
        returns ``(loss value, scores or None)``; the score matrix is written only if asked for
        (metrics).  ``loss`` is one of the objects of ``metrics`` (e.g. ``SparseSquaredHingeLoss``)."""
        if inputs.dim() != 2 or inputs.shape[1] != self.input_dim:
            raise ValueError(f"inputs must have shape [batch, {self.input_dim}], got {tuple(inputs.shape)}")
        indices = self.kernel_indices.view(-1, self.fan_in)
        weights = self.kernel_weights.view(-1, self.fan_in)
        return loss.fused(inputs.float(), indices, weights, self.bias, y_true, transposed=False, want_scores=want_scores)

    @torch.no_grad()
    def fused_train_step(self, inputs: torch.Tensor, y_true, loss, optimizer, need_input_grad: bool = False):
        """Forward, loss, backward and the Adam step on this layer's variables in two library calls: the
        forward kernel stores loss gradients (non-zero ones only) instead of scores, the backward pass
        walks them and the Adam pass skips the gradient rows of labels that received none.  ``optimizer`` is a
        ``SparseAdam`` that owns ``kernel_weights`` (and ``bias``); this uses its moments and
        ``iterations + 1`` as the step number and leaves ``optimizer.step()`` (other parameters, the
        counter) to the caller.  Returns ``(loss value, gradient with respect to inputs or None)``."""
        from . import metrics, optimizer as opt_mod
        if inputs.dim() != 2 or inputs.shape[1] != self.input_dim:
            raise ValueError(f"inputs must have shape [batch, {self.input_dim}], got {tuple(inputs.shape)}")
        inputs = inputs.float().contiguous()
        indices = self.kernel_indices.view(-1, self.fan_in)
        weights = self.kernel_weights.data.view(-1, self.fan_in)
        bias = self.bias.data if self.use_bias else None
        _, out_grad, loss_sum, masks = metrics.forward_loss(inputs, indices, weights, bias, y_true, loss.kind, want_masks=True,
                                                            skip_zero_stores=True)
        iw = optimizer._index_of(self.kernel_weights)
        ib = optimizer._index_of(self.bias) if self.use_bias else None
        input_grad, _ = opt_mod.backward_sparse_adam(
            inputs, indices, weights, out_grad, masks, optimizer._momentums[iw], optimizer._velocities[iw],
            bias, optimizer._momentums[ib] if self.use_bias else None, optimizer._velocities[ib] if self.use_bias else None,
            optimizer.learning_rate, optimizer.beta_1, optimizer.beta_2, optimizer.epsilon, optimizer.iterations + 1,
            grad_is_partial=True, need_feature_grad=need_input_grad, decide_from_previous=True)
        return loss_sum[0] / (inputs.shape[0] * self.units), input_grad

    # sparse/layer.py:215-219, 236-237 and sparse/custom_layer.py:20-43
    @torch.no_grad()
    def rewire(self, other_vars=None):
        """Gives the selected connections new random sources (weights keep their values) and
        returns ``other_vars`` (e.g. Adam moments, sparse/optimizer.py:14-23) with the entries at
        the rewired locations set to zero.  The index buffer is edited in place and the library is
        told so: it rebuilds its plan before the next backward call."""
        other_vars = [] if other_vars is None else list(other_vars)
        self._rewire_count += 1
        if hasattr(self.rewire_selector, "threshold_tensor"):
            # selection, redraw and clearing in the library: one threshold (radix select), one pass over the variables
            threshold = self.rewire_selector.threshold_tensor(self.kernel_weights.detach())
            outputs = [other.clone().contiguous() for other in other_vars]
            ops.rewire_connections(self.kernel_indices, self.kernel_weights.detach().contiguous(), [o.view(-1) for o in outputs],
                                   self.input_dim, threshold, self._rewire_seed + self._rewire_count)
        else:
            # a selector that only offers a boolean mask: the same steps as torch index operations
            locations = torch.nonzero(self.rewire_selector.select(self.kernel_weights.detach())).reshape(-1)
            if locations.numel():
                self.kernel_indices[locations] = self._random_sources(locations.numel(), self.kernel_indices.device)
            if self.kernel_indices.is_cuda:
                ops.lookup_edited(self.kernel_indices)
            outputs = []
            for other in other_vars:
                new_v = other.clone()
                new_v.reshape(-1)[locations] = 0
                outputs.append(new_v)
        if self.arrange:
            self.arrange_connections(outputs)
        return outputs


class StratifiedRewireLayer(StratifiedRewireLayerV2):
    """The reference's first fixed-fan-in layer (sparse/layer.py:339-390): the same variables and the same
    arithmetic as ``StratifiedRewireLayerV2`` (there a ``tf.sparse`` product with a kernel whose rows all hold
    ``connections // units`` entries), with one visible difference: every rewiring re-sorts the connections
    (``tf.sparse.reorder``), so inside a unit the sources are in ascending order, and weights and optimizer state
    move with them.  Here the call runs through the same fixed-fan-in kernels; sorted rows are also the layout the
    inference configuration gathers fastest."""

    def __init__(self, units: int, input_dim: int, **kwargs):
        kwargs["arrange"] = False          # the order inside a unit is this layer's own
        super().__init__(units, input_dim, **kwargs)
        # sorted from construction on, as build() leaves the reference's kernel (sparse/layer.py:197: _update_sparse_kernel
        # runs tf.sparse.reorder)
        self._sort_rows([])

    @torch.no_grad()
    def _sort_rows(self, other_vars):
        idx = self.kernel_indices.view(-1, self.fan_in)
        order = torch.argsort(idx.to(torch.int64), dim=1, stable=True)
        self.kernel_indices.copy_(torch.gather(idx, 1, order).reshape(-1))
        if self.kernel_indices.is_cuda:
            ops.lookup_edited(self.kernel_indices)
        self.kernel_weights.data.copy_(torch.gather(self.kernel_weights.data.view(-1, self.fan_in), 1, order).reshape(-1))
        return [torch.gather(o.reshape(-1, self.fan_in), 1, order).reshape(o.shape) for o in other_vars]

    @torch.no_grad()
    def rewire(self, other_vars=None):
        return self._sort_rows(super().rewire(other_vars))
