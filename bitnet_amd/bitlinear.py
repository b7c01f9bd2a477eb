"""Host-side mirror of the reference's BitLinear operator interface
(gpu/model.py:18-85) on top of libbitlinear_hip.so.

Same names, argument meaning and tensor layouts as the reference:
``bitnet_int8xint2_linear(input0, input1, s, ws)``, ``BitLinearKernel`` with a
packed int8 ``weight`` of shape (out_features, in_features // 4) and a 4-slot
bf16 ``weight_scale``, and the fake-quant ``BitLinear``.  torch is used for
device memory and the current stream only; all arithmetic of the int8 path
runs in the HIP library.
"""
import ctypes

import torch
from torch import nn
from torch.nn import functional as F

from . import _lib

QUANT_COMPILED = 0
QUANT_EAGER_BF16 = 1


def _ptr(t: torch.Tensor) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr())


def _stream_ptr() -> ctypes.c_void_p:
    # torch names the HIP stream handle `cuda_stream` on ROCm builds too
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check_device(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("bitlinear: all tensors must live on the GPU (no CPU path exists)")
        if not t.is_contiguous():
            raise ValueError("bitlinear: tensors must be contiguous")


def _flat_rows(input0: torch.Tensor) -> int:
    m = 1
    for d in input0.shape[:-1]:
        m *= d
    return m


def bitnet_int8xint2_linear(input0, input1, s, ws, out=None):
    """int8 activations [..., K] x packed ternary weight [N, K/4] -> bf16
    [..., N] (gpu/model.py:21-37).  ``s`` holds one bf16 scale per token row,
    ``ws`` the bf16 weight scales.  The output is allocated here with
    torch.empty unless ``out`` is given (the library writes every element, so
    the reference's zero fill is not needed)."""
    _check_device(input0, input1, s, ws)
    if input0.dtype != torch.int8 or input1.dtype != torch.int8:
        raise TypeError("input0 and input1 must be int8")
    if s.dtype != torch.bfloat16 or ws.dtype != torch.bfloat16:
        raise TypeError("s and ws must be bfloat16")
    out_shape = list(input0.shape)
    out_shape[-1] = input1.shape[0]
    M = _flat_rows(input0)
    N = input1.shape[0]
    K = input1.shape[1] * 4
    if input0.shape[-1] != K:
        raise ValueError(f"activation width {input0.shape[-1]} does not match packed weight K={K}")
    if s.numel() < M:
        raise ValueError(f"need one activation scale per row: {s.numel()} < {M}")
    lib = _lib.load_library()
    if ws.numel() < lib.bitlinear_ws_num(N, K):
        raise ValueError("weight_scale has fewer slots than this shape uses")
    if out is None:
        out = torch.empty(*out_shape, dtype=torch.bfloat16, device=input0.device)
    elif out.dtype != torch.bfloat16 or out.numel() != M * N or not out.is_contiguous() or not out.is_cuda:
        raise ValueError("out must be a contiguous bfloat16 GPU tensor of M x N elements")
    if M == 0:
        return out  # no token rows: nothing to launch
    lib.bitlinear_int8xint2(_ptr(input0), _ptr(input1), _ptr(out), _ptr(s), _ptr(ws), M, N, K, _stream_ptr())
    _lib.check(lib.bitlinear_last_status(), f"bitlinear_int8xint2(M={M}, N={N}, K={K})")
    return out


def bitnet_int8xint2_acc(input0, input1):
    """Raw int32 accumulators [..., N] of the same product (test/debug)."""
    _check_device(input0, input1)
    if input0.dtype != torch.int8 or input1.dtype != torch.int8:
        raise TypeError("input0 and input1 must be int8")
    M = _flat_rows(input0)
    N = input1.shape[0]
    K = input1.shape[1] * 4
    if input0.shape[-1] != K:
        raise ValueError(f"activation width {input0.shape[-1]} does not match packed weight K={K}")
    acc = torch.empty(*input0.shape[:-1], N, dtype=torch.int32, device=input0.device)
    if M == 0:
        return acc
    lib = _lib.load_library()
    st = lib.bitlinear_int8xint2_acc_i32(_ptr(input0), _ptr(input1), _ptr(acc), None, None, None, M, N, K, _stream_ptr())
    _lib.check(st, f"bitlinear_int8xint2_acc_i32(M={M}, N={N}, K={K})")
    return acc


def bitlinear_forward_acc(input, weight, weight_scale, mode: int = QUANT_COMPILED):
    """BitLinearKernel.forward through bitlinear_forward_bf16_acc_i32: the bf16
    output [..., N] together with the int32 accumulators of its product (test/debug)."""
    _check_device(input, weight, weight_scale)
    if input.dtype != torch.bfloat16 or weight.dtype != torch.int8 or weight_scale.dtype != torch.bfloat16:
        raise TypeError("expected bfloat16 activations, int8 packed weight, bfloat16 weight scales")
    M = _flat_rows(input)
    N = weight.shape[0]
    K = weight.shape[1] * 4
    if input.shape[-1] != K:
        raise ValueError(f"activation width {input.shape[-1]} does not match packed weight K={K}")
    lib = _lib.load_library()
    if weight_scale.numel() < lib.bitlinear_ws_num(N, K):
        raise ValueError("weight_scale has fewer slots than this shape uses")
    out = torch.empty(*input.shape[:-1], N, dtype=torch.bfloat16, device=input.device)
    acc = torch.empty(*input.shape[:-1], N, dtype=torch.int32, device=input.device)
    if M == 0:
        return out, acc
    q = torch.empty(M, K, dtype=torch.int8, device=input.device)
    s = torch.empty(M, dtype=torch.bfloat16, device=input.device)
    st = lib.bitlinear_forward_bf16_acc_i32(
        _ptr(input), _ptr(weight), _ptr(acc), _ptr(out), _ptr(weight_scale), _ptr(q), _ptr(s), M, N, K, mode, _stream_ptr()
    )
    _lib.check(st, f"bitlinear_forward_bf16_acc_i32(M={M}, N={N}, K={K})")
    return out, acc


def last_kernel() -> str:
    """Name of the product kernel the calling thread's last library call launched."""
    return _lib.load_library().bitlinear_last_kernel().decode()


def bitnet_int8xint2_linear_seg(input0, input1, s, ws, seg_ends, out=None):
    """Like bitnet_int8xint2_linear but row n takes ws[j] of the segment
    [seg_ends[j-1], seg_ends[j]) it lies in -- the scale layout
    gpu/convert_checkpoint.py:42-77 writes for fused wqkv / w13."""
    _check_device(input0, input1, s, ws)
    if input0.dtype != torch.int8 or input1.dtype != torch.int8:
        raise TypeError("input0 and input1 must be int8")
    if s.dtype != torch.bfloat16 or ws.dtype != torch.bfloat16:
        raise TypeError("s and ws must be bfloat16")
    M = _flat_rows(input0)
    N = input1.shape[0]
    K = input1.shape[1] * 4
    if input0.shape[-1] != K:
        raise ValueError(f"activation width {input0.shape[-1]} does not match packed weight K={K}")
    if s.numel() < M:
        raise ValueError(f"need one activation scale per row: {s.numel()} < {M}")
    if ws.numel() < len(seg_ends):
        raise ValueError("weight_scale has fewer slots than there are segments")
    if out is None:
        out = torch.empty(*input0.shape[:-1], N, dtype=torch.bfloat16, device=input0.device)
    elif out.dtype != torch.bfloat16 or out.numel() != M * N or not out.is_contiguous() or not out.is_cuda:
        raise ValueError("out must be a contiguous bfloat16 GPU tensor of M x N elements")
    if M == 0:
        return out
    ends = (ctypes.c_int * len(seg_ends))(*[int(e) for e in seg_ends])
    lib = _lib.load_library()
    st = lib.bitlinear_int8xint2_seg(
        _ptr(input0), _ptr(input1), _ptr(out), _ptr(s), _ptr(ws), ends, len(seg_ends), M, N, K, _stream_ptr()
    )
    _lib.check(st, f"bitlinear_int8xint2_seg(M={M}, N={N}, K={K})")
    return out


def quant_input(input, mode: int = QUANT_COMPILED):
    """Per-token absmax quantizer (gpu/model.py:68-71): bf16 [..., K] ->
    (int8 [..., K], bf16 scales [..., 1]).  One fused HIP kernel."""
    _check_device(input)
    if input.dtype != torch.bfloat16:
        raise TypeError("quant_input expects bfloat16")
    M = _flat_rows(input)
    K = input.shape[-1]
    q = torch.empty(input.shape, dtype=torch.int8, device=input.device)
    s = torch.empty(*input.shape[:-1], 1, dtype=torch.bfloat16, device=input.device)
    if M == 0:
        return q, s
    lib = _lib.load_library()
    st = lib.bitlinear_quant_absmax(_ptr(input), _ptr(q), _ptr(s), M, K, mode, _stream_ptr())
    _lib.check(st, f"bitlinear_quant_absmax(M={M}, K={K})")
    return q, s


class BitLinearKernel(nn.Module):
    """Drop-in for the reference module of the same name (gpu/model.py:54-75):
    same parameter names, shapes and dtypes, so a ``model_state_int2.pt``
    state dict loads unchanged."""

    in_features: int
    out_features: int
    weight: torch.Tensor
    weight_scale: torch.Tensor

    def __init__(self, in_features: int, out_features: int, bias: bool = False, quant_mode: int = QUANT_COMPILED,
                 seg_ends=None):
        """seg_ends (not in the reference, opt-in): the output-row boundaries of
        the sub-tensors a fused weight was assembled from, e.g. (2560, 3200,
        3840) for wqkv.  Row n then takes weight_scale[j] of the segment it
        lies in -- the layout gpu/convert_checkpoint.py:42-50 stores -- instead
        of the reference kernel's equal slots n // (N // ws_num)
        (bitnet_kernels.h:80), which hand q rows 1280..2559 the k scale."""
        super().__init__()
        if bias:
            raise ValueError("BitLinearKernel has no bias")
        self.in_features = in_features
        self.out_features = out_features
        self.quant_mode = quant_mode
        self.set_segments(seg_ends)
        self.weight = nn.Parameter(torch.zeros(out_features, in_features // 4, dtype=torch.int8), requires_grad=False)
        self.weight_scale = nn.Parameter(torch.zeros(4, dtype=torch.bfloat16), requires_grad=False)

    def set_segments(self, seg_ends) -> None:
        """Switch between the reference's equal-slot rule (None) and explicit
        output-row segments for the weight scales."""
        if seg_ends is None:
            self.seg_ends, self._seg_c = None, None
            return
        ends = tuple(int(e) for e in seg_ends)
        if not 1 <= len(ends) <= 4 or ends[-1] != self.out_features or any(b <= a for a, b in zip((0,) + ends, ends)):
            raise ValueError(f"seg_ends {ends}: 1 to 4 strictly increasing row boundaries ending at out_features")
        self.seg_ends = ends
        self._seg_c = (ctypes.c_int * len(ends))(*ends)

    def quant_input(self, input):
        return quant_input(input, self.quant_mode)

    def forward(self, input):
        _check_device(input, self.weight, self.weight_scale)
        if input.dtype != torch.bfloat16:
            raise TypeError("BitLinearKernel.forward expects bfloat16 activations")
        if input.shape[-1] != self.in_features:
            raise ValueError(f"activation width {input.shape[-1]} does not match in_features={self.in_features}")
        if self.weight.shape != (self.out_features, self.in_features // 4) or self.weight.dtype != torch.int8:
            raise ValueError("weight must be int8 [out_features, in_features // 4] (the packed layout)")
        M = _flat_rows(input)
        N, K = self.out_features, self.in_features
        q = torch.empty(input.shape, dtype=torch.int8, device=input.device)
        s = torch.empty(M, dtype=torch.bfloat16, device=input.device)
        out = torch.empty(*input.shape[:-1], N, dtype=torch.bfloat16, device=input.device)
        if M == 0:
            return out
        lib = _lib.load_library()
        if self.seg_ends is not None:
            st = lib.bitlinear_forward_bf16_seg(
                _ptr(input), _ptr(self.weight), _ptr(out), _ptr(self.weight_scale), self._seg_c, len(self.seg_ends),
                _ptr(q), _ptr(s), M, N, K, self.quant_mode, _stream_ptr(),
            )
            _lib.check(st, f"bitlinear_forward_bf16_seg(M={M}, N={N}, K={K})")
            return out
        st = lib.bitlinear_forward_bf16(
            _ptr(input), _ptr(self.weight), _ptr(out), _ptr(self.weight_scale), _ptr(q), _ptr(s), M, N, K,
            self.quant_mode, _stream_ptr(),
        )
        _lib.check(st, f"bitlinear_forward_bf16(M={M}, N={N}, K={K})")
        return out


class BitLinear(nn.Linear):
    """The reference's fake-quant fp module (gpu/model.py:77-85), kept in
    plain torch: activations are snapped to the int8 grid and multiplied with
    dequantised bf16 weights.  Used for comparisons with the int8 path."""

    def quant_input(self, input):
        s = 127 / input.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
        return (input * s).round().clamp(-128, 127) / s

    def forward(self, input):
        return F.linear(self.quant_input(input), self.weight)
