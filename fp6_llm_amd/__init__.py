"""fp6_llm_amd -- MI355X-native FP6/FP5 x FP16 linear layer behind the operator API of usyd-fsalab/fp6_llm.

Same names, argument meaning and shapes as the reference package (fp6_llm/__init__.py:1, bound in
fp6_llm/csrc/pybind.cpp:6-16):

    weight_prepacking_cpu, weight_dequant_cpu, linear_forward_cuda,
    weight_prepacking_eXmY_cpu, weight_dequant_eXmY_cpu, linear_forward_eXmY_cuda,
    Num_Wave, HeuristicFuntion_SplitK

plus what the gfx950 engine adds: the native weight layout (``weight_prepacking_native_cpu``, ``to_native``,
``linear_forward_native``), a device-side dequantizer and a split-K heuristic derived for 256 compute units.

Everything is computed by ``libfp6mi.so`` (C ABI in include/fp6mi.h).  The per-call GEMM path goes through a small torch
C++ extension over that ABI (``_fp6mi_torch``, csrc/torch_binding.cpp) when it is built, else through ctypes -- the same
library and kernels either way (``FP6MI_NO_TORCH_EXT=1`` forces ctypes); everything else uses ctypes.  Torch only owns
memory and streams.  Where the reference aborts the process (assert / exit) these functions raise ``ValueError`` /
``RuntimeError`` instead.
"""
import math
import os
import threading
import weakref

import torch

from . import _lib
from ._lib import Fp6miError  # noqa: F401

# The native library is loaded on first use (every entry point raises ImportError while it is missing: there is no other
# path), so that `python -m fp6_llm_amd.build` can import this package before anything is built.  The torch extension links
# against it and is only tried once it is there.  A library left over from an older source tree (a symbol missing) must not
# stop the import either, or the build module could not be started to replace it: the first real call reports it.
_ext = None
if os.path.exists(_lib.LIB_PATH) and not os.environ.get("FP6MI_NO_TORCH_EXT"):
    try:
        _lib.lib()
        from . import _fp6mi_torch as _ext
    except (ImportError, OSError, AttributeError):   # extension not built, or a stale library: the ctypes path reports what is wrong
        _ext = None

__all__ = [
    "linear_forward_cuda", "weight_prepacking_cpu", "weight_dequant_cpu",
    "linear_forward_eXmY_cuda", "weight_prepacking_eXmY_cpu", "weight_dequant_eXmY_cpu",
    "Num_Wave", "HeuristicFuntion_SplitK",
    "weight_prepacking_native_cpu", "to_native", "linear_forward_native", "native_bytes",
    "weight_dequant_native_cuda", "weight_quantize_native_cuda", "heuristic_splitk_mi355x", "clear_caches",
]

MI355X_CUS = 256


# ----------------------------------------------------------------------------------------------------------------
# Pure-Python heuristic of the reference, kept verbatim in behaviour (fp6_llm/__init__.py:6-23).
# ----------------------------------------------------------------------------------------------------------------
def Num_Wave(M, N, SplitK, Num_GPU_SMs):
    return math.ceil(M / 512) * math.ceil(N / 64) * SplitK / Num_GPU_SMs


def HeuristicFuntion_SplitK(M, N, Num_GPU_SMs):
    """Smallest SplitK in [1, 99] whose last wave of 512x64-output CTAs is at least 80 % full; 1 if none."""
    for i in range(1, 100):
        waves = Num_Wave(M, N, i, Num_GPU_SMs)
        if waves / math.ceil(waves) >= 0.8:
            return i
    return 1


def heuristic_splitk_mi355x(M, N, K, num_cus=MI355X_CUS, EXPONENT=3, MANTISSA=2):
    """Split-K for this engine's kernels: K is already split across the wavefronts of a workgroup, so a split across
    workgroups (second launch + FP32 workspace traffic) only pays when M/16 workgroups cannot occupy the chip.  The answer
    comes from the table measured for the format's bit width where the problem is near a measured one."""
    return _lib.lib().fp6mi_heuristic_splitk_format(EXPONENT, MANTISSA, M, N, K, num_cus)


# ----------------------------------------------------------------------------------------------------------------
# helpers
# ----------------------------------------------------------------------------------------------------------------
# FP6_e3m2 and FP5_e2m2 are the reference's formats (fp6_llm/csrc/fp6_linear.cu:133-138); FP6_e2m3 and FP4_e2m1 run through
# the same entry points here.
FORMATS = ((3, 2), (2, 2), (2, 3), (2, 1))
_BLOCK_BYTES = {6: 3072, 5: 2560, 4: 2048}   # bytes of a 16-row x 256-column block of the native layout, by bit width


def _bits(E, M):
    if (E, M) not in FORMATS:
        raise ValueError("unsupported format: EXPONENT=%d, MANTISSA=%d (only e3m2, e2m2, e2m3 and e2m1)" % (E, M))
    return 1 + E + M


def _weight_shape(t, E, M, name):
    x = _bits(E, M)
    if t.dtype != torch.int32 or t.dim() != 2:
        raise ValueError("%s must be a 2-D int32 tensor [OC, IC/32*%d]" % (name, x))
    OC, words = t.shape
    if words % x != 0:
        raise ValueError("%s.size(1)=%d is not a multiple of %d" % (name, words, x))
    return OC, words // x * 32


def _cpu_contig(t, name):
    if t.device.type != "cpu":
        raise ValueError("%s must be a CPU tensor" % name)
    return t.contiguous()


# ----------------------------------------------------------------------------------------------------------------
# CPU utilities (reference: fp6_linear.cu:211-223, 234-251, 323-341, 352-375)
# ----------------------------------------------------------------------------------------------------------------
def weight_prepacking_eXmY_cpu(EXPONENT, MANTISSA, fpx_tensor):
    """int32 CPU [OC, IC/32*x] raw codes -> same shape/dtype, the reference's prepacked layout, bit-exact."""
    OC, IC = _weight_shape(fpx_tensor, EXPONENT, MANTISSA, "fpx_tensor")
    if OC % 256 != 0 or IC % 64 != 0:
        raise ValueError("weight_prepacking: need OC %% 256 == 0 and IC %% 64 == 0, got OC=%d IC=%d" % (OC, IC))
    src = _cpu_contig(fpx_tensor, "fpx_tensor")
    out = torch.empty_like(src)
    _lib.check(_lib.lib().fp6mi_prepack_ref(EXPONENT, MANTISSA, out.data_ptr(), src.data_ptr(), OC, IC), "fp6mi_prepack_ref")
    return out


def weight_prepacking_cpu(fp6_tensor):
    return weight_prepacking_eXmY_cpu(3, 2, fp6_tensor)


def weight_dequant_eXmY_cpu(EXPONENT, MANTISSA, fpx_tensor, fp16_scale):
    """Raw (NOT prepacked) int32 CPU weights + fp16 [OC] scales -> fp16 [OC, IC], bit-exact to the reference."""
    OC, IC = _weight_shape(fpx_tensor, EXPONENT, MANTISSA, "fpx_tensor")
    if fp16_scale.dtype != torch.float16 or fp16_scale.dim() != 1 or fp16_scale.shape[0] != OC:
        raise ValueError("fp16_scale must be a float16 tensor of shape [OC]")
    src = _cpu_contig(fpx_tensor, "fpx_tensor")
    sc = _cpu_contig(fp16_scale, "fp16_scale")
    out = torch.empty((OC, IC), dtype=torch.float16)
    _lib.check(_lib.lib().fp6mi_dequant(EXPONENT, MANTISSA, out.data_ptr(), src.data_ptr(), OC, IC, sc.data_ptr()), "fp6mi_dequant")
    return out


def weight_dequant_cpu(fp6_tensor, fp16_scale):
    return weight_dequant_eXmY_cpu(3, 2, fp6_tensor, fp16_scale)


# ----------------------------------------------------------------------------------------------------------------
# native layout
# ----------------------------------------------------------------------------------------------------------------
def native_bytes(EXPONENT, MANTISSA, OC, IC):
    n = _lib.lib().fp6mi_native_bytes(EXPONENT, MANTISSA, OC, IC)
    if n == 0:
        raise ValueError("native layout needs OC % 16 == 0, IC % 64 == 0 and a supported format")
    return n


def weight_prepacking_native_cpu(EXPONENT, MANTISSA, fpx_tensor):
    """Raw int32 CPU weights -> 1-D int32 tensor holding the native gfx950 layout (K padded to 256)."""
    OC, IC = _weight_shape(fpx_tensor, EXPONENT, MANTISSA, "fpx_tensor")
    src = _cpu_contig(fpx_tensor, "fpx_tensor")
    out = torch.empty(native_bytes(EXPONENT, MANTISSA, OC, IC) // 4, dtype=torch.int32)
    _lib.check(_lib.lib().fp6mi_prepack_native(EXPONENT, MANTISSA, out.data_ptr(), src.data_ptr(), OC, IC), "fp6mi_prepack_native")
    return out


def to_native(packed_tensor, EXPONENT=3, MANTISSA=2):
    """Reference-layout weights (output of weight_prepacking*_cpu, on CPU or GPU) -> native layout on the same device.
    On a GPU the conversion is one kernel on the current stream."""
    OC, IC = _weight_shape(packed_tensor, EXPONENT, MANTISSA, "packed_tensor")
    src = packed_tensor.contiguous()
    out = torch.empty(native_bytes(EXPONENT, MANTISSA, OC, IC) // 4, dtype=torch.int32, device=src.device)
    if src.device.type == "cpu":
        _lib.check(_lib.lib().fp6mi_relayout_ref_to_native(EXPONENT, MANTISSA, out.data_ptr(), src.data_ptr(), OC, IC),
                   "fp6mi_relayout_ref_to_native")
    else:
        with torch.cuda.device(src.device):
            stream = torch.cuda.current_stream().cuda_stream
            _lib.check(_lib.lib().fp6mi_relayout_ref_to_native_gpu(EXPONENT, MANTISSA, stream, out.data_ptr(), src.data_ptr(), OC, IC),
                       "fp6mi_relayout_ref_to_native_gpu")
    return out


def group_exps_bytes(OC, IC):
    n = _lib.lib().fp6mi_group_exps_bytes(OC, IC)
    if n == 0:
        raise ValueError("group exponents need OC % 16 == 0 and IC % 64 == 0")
    return n


def pack_group_exps(exps, OC, IC):
    """Group exponents [OC, ceil(IC/128)] uint8 (factor 2^(b-127) on each group of 128 columns of a row; CPU tensor) -> the
    1-D uint8 tensor in the order the kernels read."""
    if exps.dtype != torch.uint8 or exps.dim() != 2 or exps.shape != (OC, (IC + 127) // 128) or exps.device.type != "cpu":
        raise ValueError("exps must be a CPU uint8 tensor [OC, ceil(IC/128)]")
    out = torch.empty(group_exps_bytes(OC, IC), dtype=torch.uint8)
    _lib.check(_lib.lib().fp6mi_pack_group_exps(out.data_ptr(), exps.contiguous().data_ptr(), OC, IC), "fp6mi_pack_group_exps")
    return out


def weight_dequant_grouped_cpu(EXPONENT, MANTISSA, fpx_tensor, fp16_scale, exps):
    """weight_dequant_eXmY_cpu with group exponents: fp16_rn(value * 2^(b-127) * scale[row]); exps [OC, ceil(IC/128)] uint8."""
    OC, IC = _weight_shape(fpx_tensor, EXPONENT, MANTISSA, "fpx_tensor")
    src = _cpu_contig(fpx_tensor, "fpx_tensor")
    if fp16_scale.dtype != torch.float16 or fp16_scale.numel() != OC:
        raise ValueError("fp16_scale must be float16 [OC]")
    if exps.dtype != torch.uint8 or exps.shape != (OC, (IC + 127) // 128):
        raise ValueError("exps must be uint8 [OC, ceil(IC/128)]")
    out = torch.empty((OC, IC), dtype=torch.float16)
    _lib.check(_lib.lib().fp6mi_dequant_grouped(EXPONENT, MANTISSA, out.data_ptr(), src.data_ptr(), OC, IC,
                                                _cpu_contig(fp16_scale, "fp16_scale").data_ptr(), _cpu_contig(exps, "exps").data_ptr()),
               "fp6mi_dequant_grouped")
    return out


def _check_group_exps(group_exps, OC, IC, dev):
    if group_exps.dtype != torch.uint8 or group_exps.device != dev or not group_exps.is_contiguous() or \
            group_exps.numel() != (OC // 16) * ((IC + 255) // 256) * 32:
        raise ValueError("group_exps must be the contiguous uint8 tensor of pack_group_exps(exps, OC, IC) on the weights' GPU")


def weight_dequant_native_cuda(EXPONENT, MANTISSA, native_weight, fp16_scale, OC, IC, group_exps=None):
    """Native-layout weights on the GPU -> fp16 [OC, IC] with the GEMM's own in-register conversion (bit-exact to
    weight_dequant_eXmY_cpu of the same weights; with group_exps, to weight_dequant_grouped_cpu)."""
    _bits(EXPONENT, MANTISSA)
    if native_weight.device.type != "cuda" or fp16_scale.device != native_weight.device:
        raise ValueError("native_weight and fp16_scale must be on the same GPU")
    if native_weight.numel() * native_weight.element_size() != (OC // 16) * ((IC + 255) // 256) * _BLOCK_BYTES[1 + EXPONENT + MANTISSA]:
        raise ValueError("native_weight has the wrong size for OC=%d IC=%d" % (OC, IC))
    out = torch.empty((OC, IC), dtype=torch.float16, device=native_weight.device)
    with torch.cuda.device(native_weight.device):
        stream = torch.cuda.current_stream().cuda_stream
        if group_exps is None:
            _lib.check(_lib.lib().fp6mi_dequant_native_gpu(EXPONENT, MANTISSA, stream, out.data_ptr(), native_weight.data_ptr(),
                                                           fp16_scale.contiguous().data_ptr(), OC, IC), "fp6mi_dequant_native_gpu")
        else:
            _check_group_exps(group_exps, OC, IC, native_weight.device)
            _lib.check(_lib.lib().fp6mi_dequant_native_grouped_gpu(EXPONENT, MANTISSA, stream, out.data_ptr(), native_weight.data_ptr(),
                                                                   fp16_scale.contiguous().data_ptr(), group_exps.data_ptr(), OC, IC),
                       "fp6mi_dequant_native_grouped_gpu")
    return out


_QUANT_DTYPES = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def weight_quantize_native_cuda(EXPONENT, MANTISSA, weight, group_scales=False):
    """Float weights [OC, IC] (fp16, bf16 or fp32) on the GPU -> (native-layout int32 tensor, fp16 scales [OC]) on the same GPU:
    per-row absmax scales, round to nearest with ties to the even code, clamped at the format maximum.  Gives the same
    bits as quant.quantize_rowwise + quant.pack_raw + weight_prepacking_native_cpu on the host, without leaving the device.
    group_scales=True also chooses a power-of-two factor per row and 128 columns and returns (native, scales, group_exps),
    the same bits as quant.quantize_groupwise + pack_group_exps."""
    _bits(EXPONENT, MANTISSA)
    if weight.device.type != "cuda" or weight.dim() != 2 or weight.dtype not in _QUANT_DTYPES:
        raise ValueError("weight must be a 2-D fp16, bf16 or fp32 tensor on the GPU")
    OC, IC = weight.shape
    if OC % 16 or IC % 64:
        raise ValueError("weight_quantize_native_cuda needs OC %% 16 == 0 and IC %% 64 == 0, got [%d, %d]" % (OC, IC))
    weight = weight.contiguous()
    native = torch.empty(native_bytes(EXPONENT, MANTISSA, OC, IC) // 4, dtype=torch.int32, device=weight.device)
    scales = torch.empty(OC, dtype=torch.float16, device=weight.device)
    with torch.cuda.device(weight.device):
        stream = torch.cuda.current_stream().cuda_stream
        if group_scales:
            gexp = torch.empty(group_exps_bytes(OC, IC), dtype=torch.uint8, device=weight.device)
            _lib.check(_lib.lib().fp6mi_quantize_native_grouped_gpu(EXPONENT, MANTISSA, stream, native.data_ptr(), scales.data_ptr(), gexp.data_ptr(),
                                                                    weight.data_ptr(), _QUANT_DTYPES[weight.dtype], OC, IC),
                       "fp6mi_quantize_native_grouped_gpu")
            return native, scales, gexp
        _lib.check(_lib.lib().fp6mi_quantize_native_gpu(EXPONENT, MANTISSA, stream, native.data_ptr(), scales.data_ptr(), weight.data_ptr(),
                                                        _QUANT_DTYPES[weight.dtype], OC, IC), "fp6mi_quantize_native_gpu")
    return native, scales


# ----------------------------------------------------------------------------------------------------------------
# GEMM
# ----------------------------------------------------------------------------------------------------------------
_workspaces = {}   # (device index, stream) -> float32 tensor, grown on demand
_native_cache = {}  # id(tensor) -> (weakref, version, data_ptr, E, M, native tensor)
_native_cache_lock = threading.RLock()  # (re-entrant: a weak reference's callback may fire while the lock is held)


def clear_caches():
    _workspaces.clear()
    _native_cache.clear()
    if _ext is not None:
        _ext.clear_workspaces()
        _ext.clear_twins()


def _workspace(device, stream, nbytes):
    if torch.cuda.is_current_stream_capturing():
        # memory allocated now belongs to the graph being recorded: hand it to this call only (the graph keeps it for its
        # replays) and remember nothing, or a later eager call would share scratch memory with the graph's replays
        return torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=device)
    key = (device.index, stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() * 4 < nbytes:
        ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=device)
        _workspaces[key] = ws
    return ws


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # the current stream's handle without building a Stream object


def linear_forward_native(EXPONENT, MANTISSA, in_feats, native_weight, scales, OC, splitK=1, out=None, workspace=None, group_exps=None):
    """out[B, OC] = in_feats[B, IC] @ dequant(W)^T with W in the native layout.  Enqueued on the current stream.
    group_exps: the tensor of pack_group_exps on the same GPU for weights with per-group exponents, else None."""
    if _ext is not None:
        return _ext.linear_forward_native(EXPONENT, MANTISSA, in_feats, native_weight, scales, OC, int(splitK), out, workspace, group_exps)
    _bits(EXPONENT, MANTISSA)
    if in_feats.dtype != torch.float16 or in_feats.dim() != 2:
        raise ValueError("in_feats must be a 2-D float16 tensor [B, IC]")
    if in_feats.device.type != "cuda":
        raise ValueError("in_feats must be on the GPU")
    dev = in_feats.device
    if native_weight.device != dev or scales.device != dev:
        raise ValueError("in_feats, weights and scales must be on the same GPU")
    if scales.dtype != torch.float16 or scales.numel() != OC:
        raise ValueError("scales must be float16 [OC]")
    B, IC = in_feats.shape
    if OC % 256 != 0 or IC % 64 != 0 or B < 1:
        raise ValueError("need OC %% 256 == 0, IC %% 64 == 0, B >= 1 (got OC=%d IC=%d B=%d)" % (OC, IC, B))
    # same value as fp6mi_native_bytes, computed here: this function is on the per-token path and a 5 us kernel deserves a
    # wrapper that costs less than it does
    if native_weight.numel() * native_weight.element_size() != (OC // 16) * ((IC + 255) // 256) * _BLOCK_BYTES[1 + EXPONENT + MANTISSA]:
        raise ValueError("native_weight has the wrong size for OC=%d IC=%d" % (OC, IC))
    splitK = int(splitK)
    if splitK < 1:
        raise ValueError("splitK must be >= 1")
    x = in_feats if in_feats.is_contiguous() else in_feats.contiguous()
    sc = scales if scales.is_contiguous() else scales.contiguous()
    if out is None:
        out = torch.empty((B, OC), dtype=torch.float16, device=dev)
    elif out.shape != (B, OC) or out.dtype != torch.float16 or not out.is_contiguous() or out.device != dev:
        raise ValueError("out must be a contiguous float16 [B, OC] tensor on the same GPU")
    L = _lib.lib()
    switch = dev.index is not None and dev.index != torch.cuda.current_device()
    if switch:
        prev = torch.cuda.current_device()
        torch.cuda.set_device(dev)
    try:
        stream = _raw_stream(dev.index) if _raw_stream is not None and dev.index is not None else torch.cuda.current_stream().cuda_stream
        ws_ptr = None
        if splitK > 1:
            need = 4 * splitK * OC * B
            if workspace is None:
                workspace = _workspace(dev, stream, need)
            elif workspace.dtype != torch.float32 or workspace.numel() * 4 < need or workspace.device != dev:
                raise ValueError("workspace must be a float32 GPU tensor with at least splitK*B*OC elements")
            ws_ptr = workspace.data_ptr()
        if group_exps is None:
            rc = L.fp6mi_linear_native(EXPONENT, MANTISSA, stream, native_weight.data_ptr(), sc.data_ptr(), x.data_ptr(),
                                       out.data_ptr(), OC, B, IC, ws_ptr, splitK)
        else:
            _check_group_exps(group_exps, OC, IC, dev)
            rc = L.fp6mi_linear_native_grouped(EXPONENT, MANTISSA, stream, native_weight.data_ptr(), sc.data_ptr(), group_exps.data_ptr(),
                                               x.data_ptr(), out.data_ptr(), OC, B, IC, ws_ptr, splitK)
    finally:
        if switch:
            torch.cuda.set_device(prev)
    if rc != 0:
        _lib.check(rc, "fp6mi_linear_native")
    return out


def _native_of(weights, E, M):
    """Native-layout twin of a reference-layout GPU tensor, converted once and remembered while the tensor is alive
    and unmodified (tensor identity, storage address and in-place version counter must all match).  The twin is published
    only once it is completely written: the one-time conversion waits for its kernel, so a later call on any stream or thread
    may use it without further ordering.  A first use while the current stream is being captured publishes nothing: there the
    conversion is only recorded, its result lives in the graph's memory pool and is written by every replay, so the captured
    GEMM gets a twin of its own and an eager call before the first replay converts for itself."""
    key = id(weights)
    with _native_cache_lock:
        hit = _native_cache.get(key)
        if hit is not None:
            ref, version, ptr, e, m, native = hit
            if ref() is weights and version == weights._version and ptr == weights.data_ptr() and (e, m) == (E, M):
                return native
        capturing = weights.device.type == "cuda" and torch.cuda.is_current_stream_capturing()
        native = to_native(weights, E, M)
        if capturing:
            return native
        if weights.device.type == "cuda":
            torch.cuda.current_stream(weights.device).synchronize()
        _native_cache[key] = (weakref.ref(weights, lambda _r, k=key: _native_cache.pop(k, None)), weights._version,
                              weights.data_ptr(), E, M, native)
        return native


def _sort_forward_args(a, b, c):
    """The reference code takes (in_feats, weights, scales) (fp6_linear.cu:161-165) while its README documents
    (weights, scales, in_feats) (README.md:86); the three tensors differ in dtype/rank, so both orders are accepted."""
    weights = [t for t in (a, b, c) if t.dtype == torch.int32]
    halves = [t for t in (a, b, c) if t.dtype == torch.float16]
    if len(weights) != 1 or len(halves) != 2:
        raise ValueError("expected one int32 weight tensor, one float16 [OC] scale tensor and one float16 [B, IC] input")
    scales = [t for t in halves if t.dim() == 1]
    feats = [t for t in halves if t.dim() == 2]
    if len(scales) != 1 or len(feats) != 1:
        raise ValueError("expected scales of shape [OC] and in_feats of shape [B, IC]")
    return feats[0], weights[0], scales[0]


def linear_forward_eXmY_cuda(EXPONENT, MANTISSA, in_feats, weights, scales, splitK=1):
    """Drop-in for fp_eXmY_linear_forward_cuda (fp6_linear.cu:269-313): `weights` is the REFERENCE prepacked layout
    (int32 [OC, IC/32*x] on the GPU).  Its native-layout twin is built by one relayout kernel on first use."""
    in_feats, weights, scales = _sort_forward_args(in_feats, weights, scales)
    OC, IC = _weight_shape(weights, EXPONENT, MANTISSA, "weights")
    if weights.device.type != "cuda":
        raise ValueError("weights must be on the GPU")
    if in_feats.shape[1] != IC:
        raise ValueError("in_feats has IC=%d but the weights have IC=%d" % (in_feats.shape[1], IC))
    if not weights.is_contiguous():
        raise ValueError("weights must be contiguous")
    native = _native_of(weights, EXPONENT, MANTISSA)
    return linear_forward_native(EXPONENT, MANTISSA, in_feats, native, scales, OC, splitK)


def linear_forward_cuda(in_feats, weights, scales, splitK=1):
    return linear_forward_eXmY_cuda(3, 2, in_feats, weights, scales, splitK)
