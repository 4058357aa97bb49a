"""Caller-side conveniences around the linear-layer path: a torch module that owns native-layout weights, and a small
on-disk container for them.  (The reference leaves both to the framework that embeds it -- DeepSpeed, README.md:19.)"""
import json
import struct

import numpy as np
import torch

from . import quant
from . import (MI355X_CUS, group_exps_bytes, heuristic_splitk_mi355x, linear_forward_native, native_bytes, pack_group_exps, to_native,
               weight_dequant_native_cuda, weight_prepacking_native_cpu, weight_quantize_native_cuda)

_MAGIC = b"FP6MI\x00\x01\x00"   # name, NUL, layout version 1, reserved


class FPxLinear(torch.nn.Module):
    """y = x @ dequant(W)^T (+ bias) with W held in the native gfx950 layout.  Weights are buffers, not parameters:
    the layer is inference-only, like the kernels."""

    # Batch size from which dequantize + FP16 library GEMM beats the mixed-input kernel on the MI355X, whatever the matrix: measured
    # through this module at 4096^2, 8192^2, 28672x8192 and 8192x28672, the route wins by 5-25 % from 3072 rows up, ties at 2048, and
    # loses below (at 1024 rows by 25-30 %).
    PREFILL_CROSSOVER = 3072

    def __init__(self, in_features, out_features, exponent=3, mantissa=2, bias=None, split_k=None, dequant_above="auto", group_scales=False):
        """group_scales: the layer also holds one exponent byte per row and 128 columns (factor 1 until weights are loaded).
        dequant_above: batch size from which forward() dequantizes the weights to a temporary fp16 matrix on the GPU and calls
        the FP16 library GEMM instead (prefill).  The mixed-input kernel wins while the GEMM is bound by weight bytes; from a
        few thousand rows the FP16 library runs 1.3-1.5 PFLOP/s against its 0.9-1.0, which pays for the dequantization pass
        (about 30 us at 8192 x 8192).  "auto" (default) = PREFILL_CROSSOVER rows; None never does (the temporary costs 2 bytes
        per weight for the duration of the call); an integer sets the threshold."""
        super().__init__()
        self.dequant_above = self.PREFILL_CROSSOVER if dequant_above == "auto" else dequant_above
        if out_features % 256 or in_features % 64:
            raise ValueError("FPxLinear needs out_features %% 256 == 0 and in_features %% 64 == 0")
        self.in_features, self.out_features = in_features, out_features
        self.exponent, self.mantissa = exponent, mantissa
        self.split_k = split_k
        self._split_cache = {}
        self.register_buffer("weight_native", torch.zeros(native_bytes(exponent, mantissa, out_features, in_features) // 4, dtype=torch.int32))
        self.register_buffer("scales", torch.ones(out_features, dtype=torch.float16))
        self.register_buffer("bias", bias)
        # per-group exponents (one byte per row and 128 columns, in the kernels' order), or None for row scales only
        self.register_buffer("group_exps", torch.full((group_exps_bytes(out_features, in_features),), 127, dtype=torch.uint8) if group_scales else None)

    @classmethod
    def from_raw(cls, raw_int32, scales, exponent=3, mantissa=2, bias=None, split_k=None):
        """raw_int32: the reference's raw weight tensor [OC, IC/32*x] (CPU); scales: float16 [OC]."""
        x = 1 + exponent + mantissa
        OC, IC = raw_int32.shape[0], raw_int32.shape[1] * 32 // x
        m = cls(IC, OC, exponent, mantissa, bias, split_k)
        m.weight_native.copy_(weight_prepacking_native_cpu(exponent, mantissa, raw_int32))
        m.scales.copy_(scales)
        return m

    @classmethod
    def from_prepacked(cls, packed_int32, scales, exponent=3, mantissa=2, bias=None, split_k=None):
        """packed_int32: output of weight_prepacking*_cpu (the reference layout), on CPU or GPU."""
        x = 1 + exponent + mantissa
        OC, IC = packed_int32.shape[0], packed_int32.shape[1] * 32 // x
        m = cls(IC, OC, exponent, mantissa, bias, split_k).to(packed_int32.device)
        m.weight_native.copy_(to_native(packed_int32, exponent, mantissa))
        m.scales.copy_(scales.to(packed_int32.device))
        return m

    @classmethod
    def from_float(cls, weight, exponent=3, mantissa=2, bias=None, split_k=None, group_scales=False):
        """Quantizes a float [OC, IC] weight row-wise (round to nearest even, absmax scales) and packs it; a weight that
        already lives on the GPU is quantized there (same bits as the host path).  group_scales=True adds a power-of-two
        factor per row and 128 columns (quant.quantize_groupwise), which the conversion instruction applies."""
        on_gpu = weight.device.type == "cuda" and weight.dtype in (torch.float16, torch.bfloat16, torch.float32)
        if group_scales and on_gpu:
            native, scales, gexp = weight_quantize_native_cuda(exponent, mantissa, weight.detach(), True)
            m = cls(weight.shape[1], weight.shape[0], exponent, mantissa, bias, split_k).to(weight.device)
            m.weight_native.copy_(native)
            m.scales.copy_(scales)
            m.group_exps = gexp
            return m
        if group_scales:
            codes, scales, exps = quant.quantize_groupwise(weight.detach().float().cpu().numpy(), exponent, mantissa)
            raw = torch.from_numpy(quant.pack_raw(codes, exponent, mantissa))
            m = cls.from_raw(raw, torch.from_numpy(scales), exponent, mantissa, bias, split_k)
            m.group_exps = pack_group_exps(torch.from_numpy(exps), weight.shape[0], weight.shape[1])
            return m.to(weight.device)
        if weight.device.type == "cuda" and weight.dtype in (torch.float16, torch.bfloat16, torch.float32):
            native, scales = weight_quantize_native_cuda(exponent, mantissa, weight.detach())
            m = cls(weight.shape[1], weight.shape[0], exponent, mantissa, bias, split_k).to(weight.device)
            m.weight_native.copy_(native)
            m.scales.copy_(scales)
            return m
        codes, scales = quant.quantize_rowwise(weight.detach().float().cpu().numpy(), exponent, mantissa)
        raw = torch.from_numpy(quant.pack_raw(codes, exponent, mantissa))
        return cls.from_raw(raw, torch.from_numpy(scales), exponent, mantissa, bias, split_k)

    @classmethod
    def fused(cls, layers, split_k=None):
        """One layer that computes several layers over the same input in a single launch (fused QKV, gate + up): its output
        is the concatenation of theirs along the feature axis.  Rows are independent in the native layout (16-row tiles
        are stored one after another), so fusing is a concatenation of the weight buffers, scales and biases."""
        layers = list(layers)
        first = layers[0]
        for l in layers:
            if (l.in_features, l.exponent, l.mantissa) != (first.in_features, first.exponent, first.mantissa):
                raise ValueError("fused layers must share in_features and the weight format")
            if (l.bias is None) != (first.bias is None):
                raise ValueError("fused layers must all have a bias or all have none")
            if l.weight_native.device != first.weight_native.device:
                raise ValueError("fused layers must live on one device")
            if (l.group_exps is None) != (first.group_exps is None):
                raise ValueError("fused layers must all have group exponents or all have none")
        bias = None if first.bias is None else torch.cat([l.bias for l in layers])
        m = cls(first.in_features, sum(l.out_features for l in layers), first.exponent, first.mantissa, bias, split_k)
        m = m.to(first.weight_native.device)
        m.weight_native.copy_(torch.cat([l.weight_native for l in layers]))
        m.scales.copy_(torch.cat([l.scales for l in layers]))
        if first.group_exps is not None:   # [row tile][K block][16][2] bytes: row tiles follow each other like the weights
            m.group_exps = torch.cat([l.group_exps for l in layers])
        return m

    def forward(self, x):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.in_features)
        if x2.dtype != torch.float16:
            x2 = x2.half()
        if self.dequant_above is not None and x2.shape[0] >= self.dequant_above:
            w16 = weight_dequant_native_cuda(self.exponent, self.mantissa, self.weight_native, self.scales, self.out_features, self.in_features,
                                             self.group_exps)
            y = torch.nn.functional.linear(x2, w16)
            del w16
            if self.bias is not None:
                y = y + self.bias
            return y.reshape(*lead, self.out_features)
        sk = self.split_k
        if not sk:   # the heuristic's answer per batch size is remembered: the layer is called once per token
            sk = self._split_cache.get(x2.shape[0])
            if sk is None:
                sk = self._split_cache[x2.shape[0]] = heuristic_splitk_mi355x(self.out_features, x2.shape[0], self.in_features, MI355X_CUS, self.exponent, self.mantissa)
        y = linear_forward_native(self.exponent, self.mantissa, x2, self.weight_native, self.scales, self.out_features, sk, None, None, self.group_exps)
        if self.bias is not None:
            y = y + self.bias
        return y.reshape(*lead, self.out_features)

    def extra_repr(self):
        return "in_features=%d, out_features=%d, format=e%dm%d" % (self.in_features, self.out_features, self.exponent, self.mantissa)


def save_native(path, native_int32, scales, exponent, mantissa, out_features, in_features, group_exps=None):
    """One weight matrix in the native layout: magic, little-endian uint32 header length, JSON header, native bytes, fp16 scales,
    then the packed group exponents if the weight has them."""
    nat = native_int32.detach().cpu().contiguous().numpy()
    sc = scales.detach().cpu().contiguous().numpy().astype(np.float16)
    if nat.nbytes != native_bytes(exponent, mantissa, out_features, in_features) or sc.shape != (out_features,):
        raise ValueError("buffers do not match the stated shape")
    ge = None
    if group_exps is not None:
        ge = group_exps.detach().cpu().contiguous().numpy()
        if ge.dtype != np.uint8 or ge.size != group_exps_bytes(out_features, in_features):
            raise ValueError("group_exps does not match the stated shape")
    header = json.dumps({"exponent": exponent, "mantissa": mantissa, "out_features": out_features, "in_features": in_features,
                         "layout": "native-v1", "native_bytes": int(nat.nbytes), "group_exps_bytes": 0 if ge is None else int(ge.size)}).encode()
    with open(path, "wb") as f:
        f.write(_MAGIC)
        f.write(struct.pack("<I", len(header)))
        f.write(header)
        f.write(nat.tobytes())
        f.write(sc.tobytes())
        if ge is not None:
            f.write(ge.tobytes())


def load_native(path):
    """Returns (native int32 tensor, float16 scales, header dict); the packed group exponents, if the file has them, are
    hdr["group_exps"] (uint8 tensor).  Plain binary parsing; nothing in the file is executed."""
    with open(path, "rb") as f:
        if f.read(len(_MAGIC)) != _MAGIC:
            raise ValueError("%s is not a native FPx weight file (or has another layout version)" % path)
        (hlen,) = struct.unpack("<I", f.read(4))
        if hlen > 1 << 16:
            raise ValueError("implausible header length")
        hdr = json.loads(f.read(hlen).decode())
        want = native_bytes(hdr["exponent"], hdr["mantissa"], hdr["out_features"], hdr["in_features"])
        if hdr.get("layout") != "native-v1" or hdr.get("native_bytes") != want:
            raise ValueError("header does not describe a native-v1 weight of that shape")
        nat = np.frombuffer(f.read(want), dtype=np.int32)
        sc = np.frombuffer(f.read(2 * hdr["out_features"]), dtype=np.float16)
        if nat.nbytes != want or sc.size != hdr["out_features"]:
            raise ValueError("file is truncated")
        gbytes = int(hdr.get("group_exps_bytes", 0))
        if gbytes:
            if gbytes != group_exps_bytes(hdr["out_features"], hdr["in_features"]):
                raise ValueError("header does not describe the group exponents of that shape")
            ge = np.frombuffer(f.read(gbytes), dtype=np.uint8)
            if ge.size != gbytes:
                raise ValueError("file is truncated")
            hdr["group_exps"] = torch.from_numpy(ge.copy())
    return torch.from_numpy(nat.copy()), torch.from_numpy(sc.copy()), hdr
