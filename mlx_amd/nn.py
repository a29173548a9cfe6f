"""Callers of the quantized-matmul path: the layers of
``python/mlx/nn/layers/quantized.py`` (``QuantizedLinear`` :205-307,
``QuantizedEmbedding`` :103-202, ``quantize`` :27-100) over this package's
operators.

The host module system is ``torch.nn`` (torch is the device-memory plumbing of
this package): a quantized layer keeps ``weight`` (uint32 codes), ``scales`` and
``biases`` as buffers -- frozen, as in MLX -- and an optional trainable-free
``bias``.  In the floating-point modes (``mxfp4``, ``mxfp8``, ``nvfp4``) there
are no ``biases`` and ``scales`` are bytes; ``QQLinear`` (:310-432) quantizes its
input as well.
"""
from __future__ import annotations

import math
from typing import Callable, List, Optional, Tuple, Union

import torch

from . import ops

__all__ = ["QuantizedLinear", "QQLinear", "QuantizedEmbedding", "QuantizedSwitchLinear", "SwitchGLU",
           "quantize", "save_weights", "load_weights"]


def _defaults_for_mode(mode: str, group_size: Optional[int], bits: Optional[int]):
    # python/mlx/nn/layers/quantized.py:12-24
    mode_defaults = {"affine": (64, 4), "mxfp4": (32, 4), "nvfp4": (16, 4), "mxfp8": (32, 8)}
    if mode not in mode_defaults:
        raise ValueError(
            f"Invalid quantization mode '{mode}'. Valid modes are: {', '.join(mode_defaults)}."
        )
    default_group_size, default_bits = mode_defaults[mode]
    return group_size or default_group_size, bits or default_bits


class QuantizedLinear(torch.nn.Module):
    """``y = quantized_matmul(x, weight, scales, biases, transpose=True) + bias``."""

    def __init__(self, input_dims: int, output_dims: int, bias: bool = True,
                 group_size: Optional[int] = None, bits: Optional[int] = None,
                 mode: str = "affine", device=None, dtype=torch.float32):
        super().__init__()
        self.group_size, self.bits = _defaults_for_mode(mode, group_size, bits)
        self.mode = mode
        device = torch.device("cuda:0") if device is None else torch.device(device)
        scale = math.sqrt(1.0 / input_dims)
        weight = (torch.rand((output_dims, input_dims), device=device) * 2 - 1) * scale
        self._set_quantized(weight.to(dtype))
        self.register_buffer(
            "bias", torch.zeros((output_dims,), device=device, dtype=dtype) if bias else None)

    def _set_quantized(self, weight: torch.Tensor) -> None:
        wq, scales, *biases = ops.quantize(weight, self.group_size, self.bits, self.mode)
        biases = biases[0] if biases else None  # none in the floating-point modes
        for name, t in (("weight", wq), ("scales", scales), ("biases", biases)):
            if name in self._buffers:
                self._buffers[name] = t
            else:
                self.register_buffer(name, t)

    def extra_repr(self) -> str:
        out_dims, in_dims = self.weight.shape
        in_dims = (in_dims * 32) // self.bits
        return (f"input_dims={in_dims}, output_dims={out_dims}, bias={self.bias is not None}, "
                f"group_size={self.group_size}, bits={self.bits}, mode={self.mode}")

    def prepack(self) -> "QuantizedLinear":
        """Keeps the transposed image of scales and biases that prefill calls
        (512 rows of x and more) would otherwise rebuild on every call.  Not in
        the reference; call again after changing the weights."""
        if self.mode != "affine":
            return self  # no biases, nothing to transpose
        self._sb_image = ops.quantized_matmul_sb_image(self.scales, self.biases, self.group_size)
        self._sb_image_of = (self.scales.data_ptr(), self.biases.data_ptr())
        return self

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        image = getattr(self, "_sb_image", None)
        if image is not None and (
                self.biases is None
                or self._sb_image_of != (self.scales.data_ptr(), self.biases.data_ptr())
                or torch.promote_types(x.dtype, self.scales.dtype) != image.dtype):
            image = None  # weights replaced, or a product in another type
        y = ops.quantized_matmul(x, self.weight, self.scales, self.biases, transpose=True,
                                 group_size=self.group_size, bits=self.bits, mode=self.mode,
                                 sb_image=image)
        if self.bias is not None:
            y = y + self.bias
        return y

    @classmethod
    def from_linear(cls, linear_layer, group_size: Optional[int] = None,
                    bits: Optional[int] = None, mode: str = "affine") -> "QuantizedLinear":
        output_dims, input_dims = linear_layer.weight.shape
        w = linear_layer.weight.detach()
        ql = cls(input_dims, output_dims, False, group_size, bits, mode,
                 device=w.device, dtype=w.dtype)
        ql._set_quantized(w)
        if getattr(linear_layer, "bias", None) is not None:
            ql._buffers["bias"] = linear_layer.bias.detach()
        return ql


class QQLinear(torch.nn.Module):
    """``y = qqmm(x, weight, scales)``: the input is quantized on the fly as well
    (python/mlx/nn/layers/quantized.py:310-432).  In eval mode the weight is kept
    quantized with its scales; in training mode it is kept in its floating-point
    type and quantized inside every call.  Modes ``nvfp4`` (default) and
    ``mxfp8``; no bias term."""

    def __init__(self, input_dims: int, output_dims: int, group_size: Optional[int] = None,
                 bits: Optional[int] = None, mode: str = "nvfp4", device=None,
                 dtype=torch.float32):
        super().__init__()
        self.group_size, self.bits = _defaults_for_mode(mode, group_size, bits)
        self.mode = mode
        device = torch.device("cuda:0") if device is None else torch.device(device)
        scale = math.sqrt(1.0 / input_dims)
        weight = (torch.rand((output_dims, input_dims), device=device) * 2 - 1) * scale
        self.register_buffer("weight", weight.to(dtype))
        self.register_buffer("scales", None)
        self._quantized = False

    def extra_repr(self) -> str:
        out_dims, in_dims = self.weight.shape
        if self.weight.dtype == torch.uint32:
            in_dims = (in_dims * 32) // self.bits
        return (f"input_dims={in_dims}, output_dims={out_dims}, "
                f"group_size={self.group_size}, bits={self.bits}, mode={self.mode}")

    def quantize(self) -> None:
        if not self._quantized:
            self._float_dtype = self.weight.dtype
            wq, scales = ops.quantize(self.weight, self.group_size, self.bits, self.mode)
            self._buffers["weight"], self._buffers["scales"] = wq, scales
            self._quantized = True

    def dequantize(self) -> None:
        if self._quantized:
            self._buffers["weight"] = ops.dequantize(
                self.weight, self.scales, group_size=self.group_size, bits=self.bits,
                mode=self.mode, dtype=getattr(self, "_float_dtype", None))
            self._buffers["scales"] = None
            self._quantized = False

    def train(self, mode: bool = True):
        super().train(mode)
        if mode:
            self.dequantize()
        else:
            self.quantize()
        return self

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.qqmm(x, self.weight, self.scales, group_size=self.group_size,
                        bits=self.bits, mode=self.mode)

    @classmethod
    def from_linear(cls, linear_layer, group_size: Optional[int] = None,
                    bits: Optional[int] = None, mode: str = "nvfp4") -> "QQLinear":
        output_dims, input_dims = linear_layer.weight.shape
        if getattr(linear_layer, "bias", None) is not None:
            raise NotImplementedError("QQLinear does not support bias yet.")
        w = linear_layer.weight.detach()
        ql = cls(input_dims, output_dims, group_size, bits, mode, device=w.device, dtype=w.dtype)
        ql._buffers["weight"] = w
        ql.train(linear_layer.training)
        return ql


class QuantizedEmbedding(torch.nn.Module):
    """Embedding with a quantized table: a lookup dequantizes the selected rows;
    ``as_linear`` uses the table as an output projection (tied weights)."""

    def __init__(self, num_embeddings: int, dims: int, group_size: Optional[int] = None,
                 bits: Optional[int] = None, mode: str = "affine", device=None,
                 dtype=torch.float32):
        super().__init__()
        self.group_size, self.bits = _defaults_for_mode(mode, group_size, bits)
        self.mode = mode
        self.num_embeddings, self.dims = num_embeddings, dims
        device = torch.device("cuda:0") if device is None else torch.device(device)
        weight = torch.randn((num_embeddings, dims), device=device) * math.sqrt(1.0 / dims)
        self._set_quantized(weight.to(dtype))

    _set_quantized = QuantizedLinear._set_quantized

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # torch cannot index uint32 tensors: gather the rows through an int32 view
        rows = self.weight.view(torch.int32)[x].view(torch.uint32)
        return ops.dequantize(rows, self.scales[x], None if self.biases is None else self.biases[x],
                              group_size=self.group_size, bits=self.bits, mode=self.mode)

    def as_linear(self, x: torch.Tensor) -> torch.Tensor:
        return ops.quantized_matmul(x, self.weight, self.scales, self.biases, transpose=True,
                                    group_size=self.group_size, bits=self.bits, mode=self.mode)

    def extra_repr(self) -> str:
        return (f"{self.num_embeddings}, {self.dims}, group_size={self.group_size}, "
                f"bits={self.bits}, mode={self.mode}")

    @classmethod
    def from_embedding(cls, embedding_layer, group_size: Optional[int] = None,
                       bits: Optional[int] = None, mode: str = "affine") -> "QuantizedEmbedding":
        num, dims = embedding_layer.weight.shape
        w = embedding_layer.weight.detach()
        ql = cls(num, dims, group_size, bits, mode, device=w.device, dtype=w.dtype)
        ql._set_quantized(w)
        return ql


class SwiGLU(torch.nn.Module):
    """Gated MLP block ``down(silu(gate(x)) * up(x))`` over three
    :class:`QuantizedLinear` layers (the MLP of Llama-style models built from
    ``nn.QuantizedLinear``, python/mlx/nn/layers/quantized.py:205-307).  With at
    most 8 rows of x and no additive biases the gate and up projections and the
    gate arithmetic run as one ``quantized_swiglu`` call; otherwise as the three
    separate products."""

    def __init__(self, input_dims: int, hidden_dims: int, bias: bool = False,
                 group_size: Optional[int] = None, bits: Optional[int] = None,
                 device=None, dtype=torch.float32):
        super().__init__()
        kw = dict(bias=bias, group_size=group_size, bits=bits, device=device, dtype=dtype)
        self.gate_proj = QuantizedLinear(input_dims, hidden_dims, **kw)
        self.up_proj = QuantizedLinear(input_dims, hidden_dims, **kw)
        self.down_proj = QuantizedLinear(hidden_dims, input_dims, **kw)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        g, u = self.gate_proj, self.up_proj
        rows = x.numel() // max(x.shape[-1], 1)
        fused = (0 < rows <= 8 and g.bias is None and u.bias is None
                 and (g.group_size, g.bits, g.mode) == (u.group_size, u.bits, "affine")
                 and u.mode == "affine")
        if fused:
            h = ops.quantized_swiglu(x, (g.weight, g.scales, g.biases),
                                     (u.weight, u.scales, u.biases), g.group_size, g.bits)
        else:
            h = torch.nn.functional.silu(g(x)) * u(x)
        return self.down_proj(h)


class QuantizedSwitchLinear(torch.nn.Module):
    """A stack of ``num_experts`` quantized linear layers evaluated through
    ``gather_qmm``: ``y[..., i, :, :] = x[..., :, :] @ dequant(weight[indices[..., i]]).T``
    (the expert-routed caller of the path, built on mlx/ops.cpp:5553-5629; x is
    ``[..., 1 | k, M, input_dims]`` and ``indices`` ``[..., k]``).  With
    ``sorted_indices`` the caller promises ascending indices, which lets the
    kernel group the rows of each expert."""

    def __init__(self, input_dims: int, output_dims: int, num_experts: int, bias: bool = True,
                 group_size: Optional[int] = None, bits: Optional[int] = None,
                 mode: str = "affine", device=None, dtype=torch.float32):
        super().__init__()
        self.group_size, self.bits = _defaults_for_mode(mode, group_size, bits)
        self.mode = mode
        device = torch.device("cuda:0") if device is None else torch.device(device)
        scale = math.sqrt(1.0 / input_dims)
        weight = (torch.rand((num_experts, output_dims, input_dims), device=device) * 2 - 1) * scale
        self._set_quantized(weight.to(dtype))
        self.register_buffer(
            "bias", torch.zeros((num_experts, output_dims), device=device, dtype=dtype) if bias else None)

    _set_quantized = QuantizedLinear._set_quantized

    @property
    def num_experts(self) -> int:
        return self.weight.shape[0]

    def forward(self, x: torch.Tensor, indices: torch.Tensor, sorted_indices: bool = False) -> torch.Tensor:
        y = ops.gather_qmm(x, self.weight, self.scales, self.biases, rhs_indices=indices,
                           transpose=True, group_size=self.group_size, bits=self.bits,
                           mode=self.mode, sorted_indices=sorted_indices)
        if self.bias is not None:
            y = y + self.bias[indices.long()].unsqueeze(-2)
        return y

    def extra_repr(self) -> str:
        e, out_dims, in_dims = self.weight.shape
        return (f"input_dims={in_dims * 32 // self.bits}, output_dims={out_dims}, num_experts={e}, "
                f"bias={self.bias is not None}, group_size={self.group_size}, bits={self.bits}")


class SwitchGLU(torch.nn.Module):
    """Expert-routed gated MLP: ``down(act(gate(x)) * up(x))`` with every
    projection a :class:`QuantizedSwitchLinear` and token ``t`` sent to the
    experts ``indices[t, :]``.  From 64 routed rows on, the rows are ordered by
    expert first (one argsort), so that all three projections run with
    ``sorted_indices=True``, and put back afterwards."""

    def __init__(self, input_dims: int, hidden_dims: int, num_experts: int,
                 activation: Callable[[torch.Tensor], torch.Tensor] = torch.nn.functional.silu,
                 bias: bool = False, group_size: Optional[int] = None, bits: Optional[int] = None,
                 device=None, dtype=torch.float32, sort_threshold: int = 64):
        super().__init__()
        kw = dict(bias=bias, group_size=group_size, bits=bits, device=device, dtype=dtype)
        self.gate_proj = QuantizedSwitchLinear(input_dims, hidden_dims, num_experts, **kw)
        self.up_proj = QuantizedSwitchLinear(input_dims, hidden_dims, num_experts, **kw)
        self.down_proj = QuantizedSwitchLinear(hidden_dims, input_dims, num_experts, **kw)
        self.activation = activation
        self.sort_threshold = sort_threshold

    def forward(self, x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        """x ``[..., D]``, indices ``[..., k]`` -> ``[..., k, D]``."""
        k = indices.shape[-1]
        x = x.unsqueeze(-2).unsqueeze(-3)  # [..., 1, 1, D]
        do_sort = indices.numel() >= self.sort_threshold
        idx = indices
        if do_sort:
            flat = indices.reshape(-1)
            order = torch.argsort(flat.long(), stable=True)
            inverse = torch.argsort(order)
            x = x.reshape(-1, 1, x.shape[-1])[order // k]  # [n, 1, D]: one row per routed pair
            # torch cannot index uint32 tensors: reorder through an integer copy
            idx = flat.long()[order].to(indices.dtype)
        up = self.up_proj(x, idx, sorted_indices=do_sort)
        gate = self.gate_proj(x, idx, sorted_indices=do_sort)
        y = self.down_proj(self.activation(gate) * up, idx, sorted_indices=do_sort)
        if do_sort:
            y = y[inverse].reshape(*indices.shape, 1, y.shape[-1])
        return y.squeeze(-2)


def _to_quantized(m, **kwargs):
    if isinstance(m, torch.nn.Linear):
        # Linear.to_quantized, python/mlx/nn/layers/linear.py:72-107
        if kwargs.pop("quantize_input", False):
            mode = kwargs.get("mode", "affine")
            if mode not in ("nvfp4", "mxfp8"):
                raise ValueError(
                    "Quantized activations are only supported for 'nvfp4' and 'mxfp8' "
                    f"modes, got {mode}."
                )
            return QQLinear.from_linear(m, **kwargs)
        return QuantizedLinear.from_linear(m, **kwargs)
    kwargs.pop("quantize_input", None)
    if isinstance(m, torch.nn.Embedding):
        return QuantizedEmbedding.from_embedding(m, **kwargs)
    return None


def quantize(model: torch.nn.Module, group_size: Optional[int] = None,
             bits: Optional[int] = None, *, mode: str = "affine",
             quantize_input: bool = False,
             class_predicate: Optional[Callable[[str, torch.nn.Module], Union[bool, dict]]] = None):
    """Replace, in place, the ``Linear`` and ``Embedding`` leaves of ``model`` that
    the predicate accepts by their quantized counterparts (``nn.quantize``).
    ``class_predicate(path, module)`` returns a bool or a dict of parameters for
    the conversion."""
    _defaults_for_mode(mode, group_size, bits)
    quantizable = lambda m: isinstance(m, (torch.nn.Linear, torch.nn.Embedding))  # noqa: E731
    class_predicate = class_predicate or (lambda _, m: quantizable(m))
    for path, parent in list(model.named_modules()):
        for name, child in list(parent.named_children()):
            if len(list(child.children())) != 0:
                continue  # not a leaf
            full = f"{path}.{name}" if path else name
            decision = class_predicate(full, child)
            if not decision:
                continue
            if not quantizable(child):
                raise ValueError(f"Unable to quantize model of type {type(child)}")
            if isinstance(decision, bool):
                kwargs = {"group_size": group_size, "bits": bits, "mode": mode}
                if quantize_input:
                    kwargs["quantize_input"] = True
            elif isinstance(decision, dict):
                kwargs = dict(decision)
            else:
                raise ValueError("``class_predicate`` must return a bool or a dict of "
                                 "parameters to pass to ``to_quantized``")
            setattr(parent, name, _to_quantized(child, **kwargs))
    return model


def save_weights(model: torch.nn.Module, file: str) -> None:
    """``Module.save_weights`` (python/mlx/nn/layers/base.py:209-224) for the
    ``.safetensors`` format: every parameter and buffer under its dotted path, so
    a quantized layer is stored as the triplet ``weight`` (U32 codes), ``scales``,
    ``biases`` (+ ``bias``) exactly as MLX stores a quantized model, with the
    ``{"format": "mlx"}`` metadata ``mx.save_safetensors`` writes."""
    from safetensors.torch import save_file

    if not str(file).endswith(".safetensors"):
        raise ValueError(f"Unsupported file extension for {file}. Use '.safetensors'.")
    tensors = {k: v.detach().contiguous().cpu() for k, v in model.state_dict().items()}
    save_file(tensors, str(file), metadata={"format": "mlx"})


def load_weights(model: torch.nn.Module,
                 file_or_weights: Union[str, List[Tuple[str, torch.Tensor]]],
                 strict: bool = True) -> torch.nn.Module:
    """``Module.load_weights`` (python/mlx/nn/layers/base.py:123-207): update the
    model from a ``.safetensors`` file or a list of (name, tensor) pairs.  With
    ``strict`` the names must match the model's exactly and the shapes agree;
    otherwise only the names the model has are taken.  Tensors keep their stored
    dtype (a layer's ``scales`` may be float16 in the file and the model built in
    float32) and move to the device of the tensor they replace."""
    weights = file_or_weights
    if isinstance(weights, (str, bytes)) or hasattr(weights, "__fspath__"):
        from safetensors.torch import load_file

        if not str(weights).endswith(".safetensors"):
            raise ValueError(f"Unsupported file extension for {weights}. Use '.safetensors'.")
        weights = list(load_file(str(weights)).items())
    weights = list(weights)
    current = model.state_dict()
    if strict:
        new = dict(weights)
        if extras := (new.keys() - current.keys()):
            listing = ",\n".join(sorted(extras))
            raise ValueError(f"Received {len(extras)} parameters not in model: \n{listing}.")
        if missing := (current.keys() - new.keys()):
            listing = ",\n".join(sorted(missing))
            raise ValueError(f"Missing {len(missing)} parameters: \n{listing}.")
        for k, v in current.items():
            v_new = new[k]
            if not isinstance(v_new, torch.Tensor):
                raise ValueError(f"Expected a tensor but received {type(v_new)} for parameter {k}")
            if tuple(v_new.shape) != tuple(v.shape):
                raise ValueError(
                    f"Expected shape {tuple(v.shape)} but received shape {tuple(v_new.shape)} "
                    f"for parameter {k}"
                )
    for name, value in weights:
        if name not in current:
            continue
        path, _, leaf = name.rpartition(".")
        owner = model.get_submodule(path) if path else model
        value = value.to(current[name].device)
        if leaf in owner._parameters:
            owner._parameters[leaf] = torch.nn.Parameter(value, requires_grad=owner._parameters[leaf].requires_grad
                                                         and value.is_floating_point())
        else:
            owner._buffers[leaf] = value
    return model
