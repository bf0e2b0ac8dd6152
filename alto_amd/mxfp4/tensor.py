"""Weight-wrapper tensor that routes GEMMs on a wrapped weight to the MXFP4 kernels.

Mirrors ``alto/kernels/dispatch/tensor.py:53-303`` (``TrainingWeightWrapperBaseTensor`` /
``MXFP4TrainingWeightWrapperTensor``) and ``alto/kernels/dispatch/conversion.py:42-124`` (``swap_params``) without
their torchao / torchtitan dependencies: a plain ``nn.Linear`` (``F.linear``, ``mm``, ``matmul``, ``addmm``) or a
``torch._grouped_mm(A, W, offs=...)`` whose weight is wrapped picks up the low-precision path from the wrapper's
``TrainingOpConfig``; every other op sees the plain payload.  The FSDP all-gather hooks of the reference
(tensor.py:161-210) are outside this path and not provided.
"""
from __future__ import annotations

from typing import Callable, Optional

import torch
import torch.utils._pytree as pytree
from torch import nn
from torch._prims_common import suggest_memory_format

from .config import TrainingOpConfig
from .grouped_gemm import _quantize_then_mxfp_scaled_grouped_mm
from .linear import _to_mxfp4_then_scaled_mm

_ops_to_preserve_subclass = {
    torch.ops.aten.empty_like.default,
    torch.ops.aten.new_zeros.default,
    torch.ops.aten.slice.Tensor,
    torch.ops.aten.copy_.default,
    torch.ops.aten.view.default,
    torch.ops.aten.as_strided.default,
    torch.ops.aten._to_copy.default,
    torch.ops.aten._pin_memory.default,
    torch.ops.aten.split.Tensor,
    torch.ops.aten.clone.default,
    torch.ops.aten.transpose.int,
    torch.ops.aten.t.default,
}

gemm_ops = ("linear", "mm.default", "matmul.default", "addmm.default", "matmul", "mm", "addmm")


class TrainingWeightWrapperBaseTensor(torch.Tensor):
    """Wrapper subclass holding the plain weight in ``_data`` and the recipe in ``config`` (tensor.py:53-160)."""

    config: Optional[TrainingOpConfig] = None

    @staticmethod
    def __new__(cls, tensor: torch.Tensor, config: TrainingOpConfig):
        self = torch.Tensor._make_wrapper_subclass(
            cls,
            tensor.size(),
            strides=tensor.stride(),
            storage_offset=tensor.storage_offset(),
            memory_format=suggest_memory_format(tensor),
            dtype=tensor.dtype,
            layout=tensor.layout,
            device=tensor.device,
            pin_memory=tensor.is_pinned() if tensor.device.type == "cpu" else False,
            requires_grad=tensor.requires_grad,
        )
        self.config = config
        return self

    def __init__(self, tensor: torch.Tensor, config: TrainingOpConfig):
        self._data = tensor
        self.config = config

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        raise NotImplementedError(f"{cls.__name__} is a base class: use a subclass that implements a precision")

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs=None):
        config = None

        def unwrap(t):
            nonlocal config
            if config is None:
                config = t.config
            else:
                assert t.config == config, f"all wrapped tensors of one op must share a config, found {t.config} and {config}"
            return t._data

        args_u, kwargs_u = pytree.tree_map_only(TrainingWeightWrapperBaseTensor, unwrap, (args, kwargs or {}))
        assert config is not None, f"__torch_dispatch__ of {func} without a wrapped argument"
        if func == torch.ops.aten.detach.default:
            return cls(args_u[0], config)
        name = getattr(func, "__name__", str(func))
        if name in gemm_ops or name == "_grouped_mm":
            raise ValueError("a low-precision GEMM reached __torch_dispatch__: the wrapped weight must be the second "
                             "operand of linear / mm / matmul / addmm / _grouped_mm")
        out = func(*args_u, **kwargs_u)
        if func not in _ops_to_preserve_subclass:
            return out
        return pytree.tree_map_only(torch.Tensor, lambda x: cls(x, config), out)

    def __repr__(self):
        return f"{type(self).__name__}(data={self._data}, config={self.config})"

    def __tensor_flatten__(self):
        return ["_data"], {"config": self.config}

    @classmethod
    def __tensor_unflatten__(cls, inner_tensors, flatten_spec, outer_size, outer_stride):
        return cls(inner_tensors["_data"], flatten_spec["config"])

    def untyped_storage(self):
        return self._data.untyped_storage()


class MXFP4TrainingWeightWrapperTensor(TrainingWeightWrapperBaseTensor):
    """Routes ``_grouped_mm`` and the linear-like ops on a wrapped weight to the MXFP4 path (tensor.py:214-303)."""

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        name = getattr(func, "__name__", "")
        if name == "_grouped_mm":
            A, B = args[0], args[1]
            bias = kwargs.get("bias", None)
            assert not isinstance(A, cls), f"A should not be a {cls.__name__}"
            assert isinstance(B, cls), f"B should be a {cls.__name__}"
            config = B.config
            offs = kwargs.get("offs", None)
            assert A.ndim == 2 and B.ndim == 3 and offs is not None, "Only 2d x 3d with offsets is supported for now"
            assert bias is None, "Bias is not supported for now"
            assert config.precision == "mxfp4", "expected TrainingOpConfig with precision=mxfp4"
            return _quantize_then_mxfp_scaled_grouped_mm(
                A, B, offs=offs, use_2dblock_x=config.use_2dblock_x, use_2dblock_w=config.use_2dblock_w,
                use_sr_grad=config.use_sr_grad, use_dge=config.use_dge, use_hadamard=config.use_hadamard,
                clip_mode=config.clip_mode, use_macro_block_scaling=config.two_level_scaling == "blockwise",
                use_uos=config.use_uos)
        if name in gemm_ops:
            trans_b = name == "linear"
            if name.startswith("addmm"):
                bias, A, B = args[0], args[1], args[2]
            else:
                A, B = args[0], args[1]
                bias = args[2] if len(args) > 2 else kwargs.get("bias", None)
            assert not isinstance(A, cls), f"A should not be a {cls.__name__} for func {name}"
            assert isinstance(B, cls), f"B should be a {cls.__name__} for func {name}"
            config = B.config
            assert config.precision == "mxfp4", "expected TrainingOpConfig with precision=mxfp4"
            Y = _to_mxfp4_then_scaled_mm(
                A, B if trans_b else B.T, use_2dblock_x=config.use_2dblock_x, use_2dblock_w=config.use_2dblock_w,
                use_sr_grad=config.use_sr_grad, use_dge=config.use_dge, clip_mode=config.clip_mode,
                use_hadamard=config.use_hadamard, use_macro_block_scaling=config.two_level_scaling == "blockwise",
                use_uos=config.use_uos)
            if bias is not None:
                Y = Y + bias
            return Y
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **kwargs)


def swap_params(module: nn.Module, *, module_filter_fn: Optional[Callable[[nn.Module, str], bool]] = None,
                config: Optional[TrainingOpConfig] = None, target_parameter_name: Optional[str] = None) -> nn.Module:
    """Wrap the weights of every module that passes ``module_filter_fn(module, fqn)`` (conversion.py:42-124).

    Bias parameters are skipped unless ``target_parameter_name`` names one explicitly.
    """
    if config is None:
        raise ValueError("training op config is required")
    if config.precision != "mxfp4":
        raise ValueError(f"Unsupported training op config: {config}")
    tensor_cls = MXFP4TrainingWeightWrapperTensor

    if isinstance(module, nn.Parameter):
        if module_filter_fn is None or module_filter_fn(module, ""):
            if not isinstance(module.data, TrainingWeightWrapperBaseTensor):
                return nn.Parameter(tensor_cls(module.data, config), requires_grad=module.requires_grad)
        return module

    def visit(mod: nn.Module, fqn: str):
        for child_name, child in mod.named_children():
            visit(child, child_name if fqn == "" else f"{fqn}.{child_name}")
        if module_filter_fn is None or module_filter_fn(mod, fqn):
            for pname, param in list(mod.named_parameters(recurse=False)):
                if target_parameter_name is not None and pname != target_parameter_name:
                    continue
                if target_parameter_name is None and "bias" in pname:
                    continue
                if not isinstance(param.data, TrainingWeightWrapperBaseTensor):
                    setattr(mod, pname, nn.Parameter(tensor_cls(param.data, config), requires_grad=param.requires_grad))

    visit(module, "")
    return module


# checkpoints written with wrapped weights load under torch.load(weights_only=True) (dispatch/tensor.py:499-503)
torch.serialization.add_safe_globals([MXFP4TrainingWeightWrapperTensor])
