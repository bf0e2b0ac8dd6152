"""``torch.ops`` registration of the six operators the reference registers as ``torchtitan::*`` Triton ops
(``mxfp_quantization.py:410,487``, ``mxfp_linear.py:142``, ``cg_forward.py:200``, ``cg_backward.py:398,500``), with
shape-only fake implementations (``mxfp_quantization.py:548-585`` and the siblings in the other files) so that graphs
traced with fake tensors carry them.

Nothing is registered at import: ``register_torch_ops()`` uses this package's own namespace, and
``register_torch_ops("torchtitan")`` takes over the reference's names in a process where ALTO's Triton ops are not
loaded (a namespace can hold each name once).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import grouped_gemm as _gg
from . import linear as _lin
from . import quantization as _q
from .quantization import BLOCK_SIZE_DEFAULT

_REGISTERED = {}


def _fake_convert_to_mxfp4(data_hp, block_size=BLOCK_SIZE_DEFAULT, axis=-1, is_2d_block=False, use_sr=False, use_asm=None,
                           philox_seed=None, philox_offset=None, clip_mode="none", use_uos=False):
    xt = data_hp.transpose(axis, -1)
    shp = xt.shape
    codes = data_hp.new_empty((*shp[:-1], shp[-1] // 2), dtype=torch.uint8)
    ss = (*shp[:-2], shp[-2] // block_size, shp[-1] // block_size) if is_2d_block else (*shp[:-1], shp[-1] // block_size)
    return codes.transpose(axis, -1), data_hp.new_empty(ss, dtype=torch.uint8).transpose(axis, -1)


def _fake_convert_from_mxfp4(data_lp, scales, output_dtype=torch.float32, block_size=BLOCK_SIZE_DEFAULT, axis=-1, is_2d_block=False,
                             use_asm=None, clip_mode="none"):
    xt = data_lp.transpose(axis, -1)
    return data_lp.new_empty((*xt.shape[:-1], xt.shape[-1] * 2), dtype=output_dtype).transpose(axis, -1)


def _gemm_mn(a, b, k_pack_a, k_pack_b, trans_a, trans_b):
    M = a.shape[1] if trans_a else a.shape[0]
    if not k_pack_a:
        M *= 2
    N = b.shape[0] if trans_b else b.shape[1]
    if not k_pack_b:
        N *= 2
    return M, N


def _fake_blockwise_mxfp4_gemm(a, a_s, b, b_s, use_2dblock_a=False, use_2dblock_b=False, k_pack_a=True, k_pack_b=True, trans_a=False,
                               trans_b=False, block_size=BLOCK_SIZE_DEFAULT, output_dtype=torch.float32):
    M, N = _gemm_mn(a, b, k_pack_a, k_pack_b, trans_a, trans_b)
    return a.new_empty((M, N), dtype=output_dtype)


def _fake_grouped_forward(inputs, expert_weights, expert_indices, input_scales, weight_scales, trans_weights=True, use_2dblock_x=False,
                          use_2dblock_w=True, output_dtype=torch.bfloat16):
    N = expert_weights.shape[1] if trans_weights else expert_weights.shape[2]
    return inputs.new_empty((inputs.shape[0], N), dtype=output_dtype)


def _fake_grouped_backward_inputs(grad_output, expert_weights, expert_indices, go_scales, expert_weight_scales, trans_weights=True,
                                  use_2dblock_x=False, use_2dblock_w=True, k_pack_w=True, output_dtype=torch.bfloat16):
    # weights [E, N', K'] (trans_weights) or [E, K', N'] with one of the dims halved by the packing
    K = expert_weights.shape[2] if trans_weights else expert_weights.shape[1]
    if not k_pack_w:
        K *= 2
    return grad_output.new_empty((grad_output.shape[0], K), dtype=output_dtype)


def _fake_grouped_backward_weights(grad_output, inputs, expert_indices, num_experts, go_scales, input_scales, trans_weights=True,
                                   use_2dblock_go=False, use_2dblock_x=True, k_pack_go=True, k_pack_x=True, output_dtype=torch.bfloat16):
    N = grad_output.shape[1] if k_pack_go else grad_output.shape[1] * 2
    K = inputs.shape[1] if k_pack_x else inputs.shape[1] * 2
    shape = (num_experts, N, K) if trans_weights else (num_experts, K, N)
    return grad_output.new_empty(shape, dtype=output_dtype)


def register_torch_ops(namespace: str = "alto_amd"):
    """Define ``torch.ops.<namespace>.{convert_to_mxfp4, convert_from_mxfp4, blockwise_mxfp4_gemm,
    mxfp4_grouped_gemm_forward, mxfp4_grouped_gemm_backward_inputs, mxfp4_grouped_gemm_backward_weights}`` with the
    reference's argument lists.  Idempotent per namespace; returns the namespace object."""
    if namespace in _REGISTERED:
        return _REGISTERED[namespace]
    op = torch.library.custom_op

    @op(f"{namespace}::convert_to_mxfp4", mutates_args=())
    def convert_to_mxfp4(data_hp: torch.Tensor, block_size: int = BLOCK_SIZE_DEFAULT, axis: int = -1, is_2d_block: bool = False,
                         use_sr: bool = False, use_asm: Optional[bool] = None, philox_seed: Optional[int] = None,
                         philox_offset: Optional[int] = None, clip_mode: str = "none",
                         use_uos: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
        return _q.convert_to_mxfp4(data_hp, block_size, axis, is_2d_block, use_sr, use_asm, philox_seed, philox_offset, clip_mode, use_uos)

    @op(f"{namespace}::convert_from_mxfp4", mutates_args=())
    def convert_from_mxfp4(data_lp: torch.Tensor, scales: torch.Tensor, output_dtype: torch.dtype = torch.float32,
                           block_size: int = BLOCK_SIZE_DEFAULT, axis: int = -1, is_2d_block: bool = False,
                           use_asm: Optional[bool] = None, clip_mode: str = "none") -> torch.Tensor:
        return _q.convert_from_mxfp4(data_lp, scales, output_dtype, block_size, axis, is_2d_block, use_asm, clip_mode)

    @op(f"{namespace}::blockwise_mxfp4_gemm", mutates_args=())
    def blockwise_mxfp4_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor, use_2dblock_a: bool = False,
                             use_2dblock_b: bool = False, k_pack_a: bool = True, k_pack_b: bool = True, trans_a: bool = False,
                             trans_b: bool = False, block_size: int = BLOCK_SIZE_DEFAULT,
                             output_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        return _lin.blockwise_mxfp4_gemm(a, a_s, b, b_s, use_2dblock_a, use_2dblock_b, k_pack_a, k_pack_b, trans_a, trans_b, block_size,
                                         output_dtype)

    @op(f"{namespace}::mxfp4_grouped_gemm_forward", mutates_args=())
    def mxfp4_grouped_gemm_forward(inputs: torch.Tensor, expert_weights: torch.Tensor, expert_indices: torch.Tensor,
                                   input_scales: torch.Tensor, weight_scales: torch.Tensor, trans_weights: bool = True,
                                   use_2dblock_x: bool = False, use_2dblock_w: bool = True,
                                   output_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        return _gg.mxfp4_grouped_gemm_forward(inputs, expert_weights, expert_indices, input_scales, weight_scales, trans_weights,
                                              use_2dblock_x, use_2dblock_w, output_dtype)

    @op(f"{namespace}::mxfp4_grouped_gemm_backward_inputs", mutates_args=())
    def mxfp4_grouped_gemm_backward_inputs(grad_output: torch.Tensor, expert_weights: torch.Tensor, expert_indices: torch.Tensor,
                                           go_scales: torch.Tensor, expert_weight_scales: torch.Tensor, trans_weights: bool = True,
                                           use_2dblock_x: bool = False, use_2dblock_w: bool = True, k_pack_w: bool = True,
                                           output_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        return _gg.mxfp4_grouped_gemm_backward_inputs(grad_output, expert_weights, expert_indices, go_scales, expert_weight_scales,
                                                      trans_weights, use_2dblock_x, use_2dblock_w, k_pack_w, output_dtype)

    @op(f"{namespace}::mxfp4_grouped_gemm_backward_weights", mutates_args=())
    def mxfp4_grouped_gemm_backward_weights(grad_output: torch.Tensor, inputs: torch.Tensor, expert_indices: torch.Tensor, num_experts: int,
                                            go_scales: torch.Tensor, input_scales: torch.Tensor, trans_weights: bool = True,
                                            use_2dblock_go: bool = False, use_2dblock_x: bool = True, k_pack_go: bool = True,
                                            k_pack_x: bool = True, output_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        return _gg.mxfp4_grouped_gemm_backward_weights(grad_output, inputs, expert_indices, num_experts, go_scales, input_scales,
                                                       trans_weights, use_2dblock_go, use_2dblock_x, k_pack_go, k_pack_x, output_dtype)

    convert_to_mxfp4.register_fake(_fake_convert_to_mxfp4)
    convert_from_mxfp4.register_fake(_fake_convert_from_mxfp4)
    blockwise_mxfp4_gemm.register_fake(_fake_blockwise_mxfp4_gemm)
    mxfp4_grouped_gemm_forward.register_fake(_fake_grouped_forward)
    mxfp4_grouped_gemm_backward_inputs.register_fake(_fake_grouped_backward_inputs)
    mxfp4_grouped_gemm_backward_weights.register_fake(_fake_grouped_backward_weights)
    _REGISTERED[namespace] = getattr(torch.ops, namespace)
    return _REGISTERED[namespace]
