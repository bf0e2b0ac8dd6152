"""Small helpers shared by the host wrappers: device checks, pointers, stream, random bits."""
from __future__ import annotations

import os
from typing import Callable, Optional

import torch

from .. import _lib

DT_BF16, DT_F32 = 0, 1
ROUND_RNE, ROUND_SR = 0, 1
CLIP = {"none": 0, "static": 1, "dynamic": 2}


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return DT_BF16
    if dt == torch.float32:
        return DT_F32
    raise AssertionError(f"unsupported dtype {dt}: only bfloat16 and float32")


def require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "alto_amd.mxfp4 runs on MI355X only: got a tensor on device "
                f"'{t.device}'. There is no CPU fallback for the HIP kernels.")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def lib():
    return _lib.load()


# ---------------------------------------------------------------------------------------------- random bits
# Stochastic rounding consumes 32 random bits per element.  By default the library's Philox4x32-10 kernel fills them;
# tests and runs that want their own bits install a source.
_rand_source: Optional[Callable[[torch.Size, torch.device], torch.Tensor]] = None


def set_rand_bits_source(fn: Optional[Callable[[torch.Size, torch.device], torch.Tensor]]) -> None:
    """Install ``fn(shape, device) -> int32 tensor`` as the source of stochastic-rounding bits (None restores the default)."""
    global _rand_source
    _rand_source = fn


# The reference picks the gfx950 hardware converts whenever ``use_asm`` is left at None (mxfp_quantization.py:426-427:
# USE_ASM = is_cdna4()); this library runs on gfx950 only, so None means the hardware converts here as well.  The switch
# below moves that default to the exact software rule of triton_fp4_ops.py:49-61 (what the reference runs on other parts
# and what its PyTorch twin restates); ``use_asm=True`` / ``False`` on a call always win, and so do explicit ``rand_bits``
# (words per element, which only the software rule consumes).
_hw_rounding_default = os.environ.get("ALTO_MXFP4_HW_SR", "1") != "0"


def use_hardware_stochastic_rounding(on: bool = True) -> None:
    """Stochastic rounding with ``use_asm=None`` (what the autograd functions pass): the hardware converts
    (``v_cvt_scalef32_sr_pk_fp4_*``, one random dword per pair of elements; the default, as in the reference on gfx950) or,
    with ``on=False``, the software rule."""
    global _hw_rounding_default
    _hw_rounding_default = bool(on)


def hardware_stochastic_rounding(use_asm: Optional[bool] = None) -> bool:
    """What a call with this ``use_asm`` rounds with.  None: the session default -- unless a source of explicit words is
    installed (``set_rand_bits_source``): only the software rule consumes those."""
    if use_asm is None:
        return _hw_rounding_default and _rand_source is None
    return bool(use_asm)


def philox_in_kernel() -> bool:
    """True when the quantizer may draw its random words itself (no source installed with ``set_rand_bits_source``)."""
    return _rand_source is None


def philox_seed_offset(seed: Optional[int], offset: Optional[int]):
    """(key, counter start) of a Philox stream: the given ones, else 63 bits from torch's CPU generator (so that
    ``torch.manual_seed`` makes a run repeatable and no device synchronisation is involved) and counter 0."""
    if seed is None:
        seed = int(torch.randint(0, 2 ** 63 - 1, (1,), dtype=torch.int64).item())
    return int(seed) & (2 ** 64 - 1), int(offset or 0) & (2 ** 64 - 1)


# A Philox stream whose (key, counter) pair lives in DEVICE memory: the quantizer reads it there and a one-thread kernel
# moves the counter on after every use.  Nothing about the random words is then a kernel argument, so a HIP graph that
# captured a stochastic-rounding quantizer draws fresh words on every replay (a host-side seed would be frozen into it).
_device_states: dict = {}
_device_state_on = False


def enable_device_philox_state(on: bool = True, seed: Optional[int] = None, device=None) -> None:
    """Switch the default source of stochastic-rounding words (calls that pass neither ``rand_bits`` nor ``philox_seed``)
    to a device-resident Philox state.  Call it BEFORE capturing a HIP graph: the state of ``device`` (default: the current
    one) is created here, with key ``seed`` (default: 63 bits from torch's CPU generator) and counter 0, because creating it
    copies from the host.  ``on=False`` returns to per-call host seeds and drops the states.  Calls the kernel cannot serve
    with its own words (``clip_mode="dynamic"``, quantisation axes other than the last two) still fill a tensor from a
    host-side seed, which a captured graph would repeat."""
    global _device_state_on
    _device_state_on = bool(on)
    _device_states.clear()
    if on:
        dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        key, _ = philox_seed_offset(seed, 0)
        _device_states[dev.index or 0] = torch.tensor([key - (1 << 64) if key >= (1 << 63) else key, 0], dtype=torch.int64, device=dev)


def philox_device_state(device: torch.device) -> Optional[torch.Tensor]:
    """The int64[2] tensor {key, counter} of ``device`` when the device-resident stream is enabled, else None."""
    if not _device_state_on:
        return None
    idx = device.index if device.index is not None else torch.cuda.current_device()
    st = _device_states.get(idx)
    if st is None:   # first use on another device: created now (not capturable; enable per device before capturing)
        key, _ = philox_seed_offset(None, 0)
        st = _device_states[idx] = torch.tensor([key, 0], dtype=torch.int64, device=torch.device("cuda", idx))
    return st


def philox_advance(state: torch.Tensor, words: int) -> None:
    """Enqueue the counter update of ``state`` past ``words`` random words on the current stream."""
    from .._lib import check
    check(lib().alto_mxfp4_philox_advance(state.data_ptr(), int(words), stream_ptr(state.device)), "alto_mxfp4_philox_advance")


def draw_rand_bits(shape, device, seed: Optional[int] = None, offset: Optional[int] = None) -> torch.Tensor:
    """32 random bits per element for stochastic rounding (int32 tensor of ``shape`` on ``device``).

    A source installed with ``set_rand_bits_source`` wins.  Otherwise the library's Philox4x32-10 kernel fills the
    tensor (``alto_mxfp4_random_bits``: memory-bound, several times faster than ``torch.randint``): key = ``seed``,
    counter start = ``offset``; without a seed, 63 bits are drawn from torch's CPU generator, so ``torch.manual_seed``
    makes a run repeatable and no device synchronisation is involved.
    """
    if _rand_source is not None:
        r = _rand_source(torch.Size(shape), device)
        assert r.shape == torch.Size(shape) and r.dtype in (torch.int32, torch.uint32)
        return r
    seed, offset = philox_seed_offset(seed, offset)
    out = torch.empty(tuple(shape), dtype=torch.int32, device=device)
    if out.numel():
        from .._lib import check
        check(lib().alto_mxfp4_random_bits(out.data_ptr(), out.numel(), int(seed) & (2 ** 64 - 1), int(offset or 0) & (2 ** 64 - 1),
                                           stream_ptr(out.device)), "alto_mxfp4_random_bits")
    return out
