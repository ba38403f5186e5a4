"""Host side of the provider: the Python stand-in for the part of Ferrule's
``CudaArtifactOperatorContext`` (crates/ferrule-backend/src/cuda/context.rs) that
drives the quantized-weight matmul path.

It owns nothing the C ABI needs to know about: torch is used only to hold device
memory and to lend a ``hipStream_t``.  Every operation fills a POD argument block
(``ferrule_amd.abi``), calls ``*_can_implement`` and then ``*_launch`` exactly as
the reference does (crates/ferrule-backend/src/cuda/cutlass.rs:1780-1812), and maps
a non-zero status to an exception the way
crates/ferrule-backend/src/cuda/cutlass.rs:2938-2963 maps it to ``Error::Internal``.

There is no CPU path here: without a GPU, or without the built library, every
operation raises.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch

from . import abi


class ProviderError(RuntimeError):
    """A native entry point returned a non-zero status."""

    def __init__(self, what: str, status: int):
        names = {abi.INVALID_ARGUMENT: "invalid argument", abi.LAUNCH_FAILED: "launch failed",
                 abi.UNSUPPORTED: "unsupported"}
        detail = ""
        if status == abi.LAUNCH_FAILED:
            detail = f", hipError_t {abi.load().ferrule_hip_last_error_code()}"
        super().__init__(f"HIP provider {what} failed: {names.get(status, 'error')} ({status}{detail})")
        self.status = status


@dataclass(frozen=True)
class HipArtifactLinearShape:
    """Counterpart of ``CudaArtifactLinearShape`` (context.rs:386-405) for the two
    quantized layouts, plus the F32-scale variant this provider adds for FP8."""

    weight_format: int            # abi.WEIGHT_FP8_E4M3 | abi.WEIGHT_MXFP4_E2M1
    out_features: int
    in_features: int
    block_m: int = 1
    block_k: int = 32
    scale_kind: int = abi.SCALE_E8M0

    @staticmethod
    def fp8_e4m3_with_e8m0_scale(out_features, in_features, block_m=128, block_k=128):
        return HipArtifactLinearShape(abi.WEIGHT_FP8_E4M3, out_features, in_features, block_m, block_k,
                                      abi.SCALE_E8M0)

    @staticmethod
    def fp8_e4m3_with_f32_scale(out_features, in_features, block_m=128, block_k=128):
        return HipArtifactLinearShape(abi.WEIGHT_FP8_E4M3, out_features, in_features, block_m, block_k,
                                      abi.SCALE_F32)

    @staticmethod
    def fp4_e2m1_packed_with_e8m0_scale(out_features, in_features):
        return HipArtifactLinearShape(abi.WEIGHT_MXFP4_E2M1, out_features, in_features, 1, 32,
                                      abi.SCALE_E8M0)

    @property
    def scale_rows(self) -> int:
        return -(-self.out_features // self.block_m)

    @property
    def scale_cols(self) -> int:
        return -(-self.in_features // self.block_k)

    def storage_lengths(self) -> tuple[int, int]:
        """(weight bytes, scale bytes) - context.rs:433-527."""
        if self.in_features == 0 or self.out_features == 0 or self.block_m == 0 or self.block_k == 0:
            raise ValueError(f"invalid HIP artifact linear shape: {self}")
        if self.weight_format == abi.WEIGHT_MXFP4_E2M1:
            if self.in_features % 32 or self.in_features % 2:
                raise ValueError(f"invalid HIP FP4 artifact linear shape: out={self.out_features} "
                                 f"in={self.in_features}")
            return self.out_features * (self.in_features // 2), self.out_features * (self.in_features // 32)
        scale_elems = self.scale_rows * self.scale_cols
        return self.out_features * self.in_features, scale_elems * (4 if self.scale_kind == abi.SCALE_F32 else 1)


@dataclass
class HipArtifactLinearHandle:
    """Device-resident weight + scale bytes (context.rs ``CudaArtifactLinearHandle``)."""

    shape: HipArtifactLinearShape
    weight: torch.Tensor   # uint8
    scale: torch.Tensor    # uint8 (E8M0) or float32


def _ptr(t: torch.Tensor | None) -> int:
    return 0 if t is None else t.data_ptr()


class HipArtifactOperatorContext:
    """One owner thread, one device, borrowed stream - as the reference's context
    (context.rs:2546-2589).  ``stream`` defaults to torch's current stream."""

    def __init__(self, device: int | str | torch.device = 0, stream: torch.cuda.Stream | None = None):
        if not torch.cuda.is_available():
            raise RuntimeError("HipArtifactOperatorContext needs a GPU (no CPU path exists)")
        self.lib = abi.load()
        self.device = torch.device("cuda", device) if isinstance(device, int) else torch.device(device)
        self._stream = stream
        self.manifest = self.lib.ferrule_hip_provider_manifest().kernel_mask
        self.kernel_launches = 0      # counterpart of CudaOpCounters.kernel_launches

    # -- plumbing ---------------------------------------------------------
    @property
    def stream(self) -> torch.cuda.Stream:
        return self._stream if self._stream is not None else torch.cuda.current_stream(self.device)

    def stream_handle(self) -> int:
        """``stream.cu_stream() as usize as u64`` (kernels.rs:547-553)."""
        return int(self.stream.cuda_stream)

    def supports(self, kernel_id: int) -> bool:
        return bool(self.manifest & abi.kernel_bit(kernel_id))

    def _two_phase(self, what: str, can_implement, launch, args) -> None:
        status = can_implement(C.byref(args))
        if status != abi.SUCCESS:
            raise ProviderError(f"validate {what}", status)
        status = launch(C.byref(args))
        if status != abi.SUCCESS:
            raise ProviderError(f"launch {what}", status)
        self.kernel_launches += 1

    # -- uploads ----------------------------------------------------------
    def upload_artifact_linear(self, shape: HipArtifactLinearShape, weight, scale) -> HipArtifactLinearHandle:
        """Copy host bytes to the device after the same length checks as
        context.rs:5049-5135."""
        wb, sb = shape.storage_lengths()
        w = torch.as_tensor(weight).contiguous().view(torch.uint8).reshape(-1)
        s = torch.as_tensor(scale).contiguous()
        s_bytes = s.numel() * s.element_size()
        if w.numel() != wb or s_bytes != sb:
            raise ValueError(f"artifact linear payload length mismatch: weight {w.numel()} vs {wb}, "
                             f"scale {s_bytes} vs {sb}")
        if shape.scale_kind == abi.SCALE_F32 and s.dtype != torch.float32:
            raise ValueError("F32 scale kind needs a float32 scale tensor")
        return HipArtifactLinearHandle(shape, w.to(self.device), s.reshape(-1).to(self.device))

    # -- decode GEMV ------------------------------------------------------
    def _gemv_args(self, handle: HipArtifactLinearHandle, x: torch.Tensor | None,
                   out: torch.Tensor, flags: int = 0) -> abi.QuantGemvArgs:
        sh = handle.shape
        a = abi.QuantGemvArgs()
        a.weight_format, a.scale_kind = sh.weight_format, sh.scale_kind
        a.batch = 0 if x is None else x.shape[0]
        a.n, a.k = sh.out_features, sh.in_features
        a.block_m, a.block_k, a.scale_cols = sh.block_m, sh.block_k, sh.scale_cols
        a.flags = flags
        a.x, a.weight, a.weight_scales, a.output = _ptr(x), _ptr(handle.weight), _ptr(handle.scale), _ptr(out)
        a.stream = self.stream_handle()
        return a

    def artifact_linear_gemv_bf16_into(self, handle: HipArtifactLinearHandle, x: torch.Tensor,
                                       out: torch.Tensor) -> torch.Tensor:
        """y[b,:] = bf16(W_dequant @ x[b,:]) for BF16 activations.  The decode
        counterpart of ``artifact_linear_matvec_into`` (context.rs:5726-5759), which
        the reference only has for f32 activations and not at all for FP4
        (context.rs:10909-10911)."""
        sh = handle.shape
        if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != sh.in_features or not x.is_contiguous():
            raise ValueError(f"linear input must be contiguous bf16 [batch, {sh.in_features}], got "
                             f"{x.dtype} {tuple(x.shape)}")
        flags = 0
        if out.dtype == torch.float32:
            flags |= abi.GEMV_OUTPUT_F32
        elif out.dtype != torch.bfloat16:
            raise ValueError("linear output must be bf16 or f32")
        if tuple(out.shape) != (x.shape[0], sh.out_features) or not out.is_contiguous():
            raise ValueError(f"linear output length mismatch: expected {(x.shape[0], sh.out_features)}, "
                             f"got {tuple(out.shape)}")
        args = self._gemv_args(handle, x, out, flags)
        self._two_phase("quantized GEMV", self.lib.ferrule_hip_quant_gemv_can_implement,
                        self.lib.ferrule_hip_quant_gemv_launch, args)
        return out

    def artifact_linear_gemv_bf16(self, handle: HipArtifactLinearHandle, x: torch.Tensor,
                                  out_dtype=torch.bfloat16) -> torch.Tensor:
        out = torch.empty((x.shape[0], handle.shape.out_features), dtype=out_dtype, device=self.device)
        return self.artifact_linear_gemv_bf16_into(handle, x, out)

    def artifact_linear_dequantize(self, handle: HipArtifactLinearHandle) -> torch.Tensor:
        """f32 [n,k] through the device converters (diagnostic / parity entry)."""
        sh = handle.shape
        out = torch.empty((sh.out_features, sh.in_features), dtype=torch.float32, device=self.device)
        args = self._gemv_args(handle, None, out)
        status = self.lib.ferrule_hip_dequant_launch(C.byref(args))
        if status != abi.SUCCESS:
            raise ProviderError("launch dequantize", status)
        self.kernel_launches += 1
        return out

    # -- drop-ins for the reference's core linear / quantize ops --------------
    def _core(self, what: str, fn, args) -> None:
        """``invoke!`` of kernels.rs:555-576: write the stream, call, map a non-zero
        hipError_t to an exception."""
        args.stream = self.stream_handle()
        status = fn(C.byref(args))
        if status != 0:
            raise ProviderError(f"core {what}", status)
        self.kernel_launches += 1

    def pack_fp8_rows_from_f32(self, values: torch.Tensor, block_size: int = 128,
                               rounding: int = abi.FP8_ROUND_CPU_REFERENCE):
        """f32 [rows, width] -> (e4m3 [rows, width], e8m0 [rows, width/block]).
        Counterpart of ``pack_fp8_rows_from_f32_preallocated`` (context.rs:10694-10741)."""
        if values.dtype != torch.float32 or values.dim() != 2 or not values.is_contiguous():
            raise ValueError("pack_fp8_rows_from_f32 expects contiguous f32 [rows, width]")
        rows, width = values.shape
        if width % block_size:
            raise ValueError(f"row width {width} is not a multiple of block {block_size}")
        packed = torch.empty((rows, width), dtype=torch.uint8, device=self.device)
        scales = torch.empty((rows, width // block_size), dtype=torch.uint8, device=self.device)
        a = abi.QuantizeArgs(kind=abi.QUANTIZE_FP8_PACKED, value_offset=0, value_len=rows * width,
                             row_width=width, block_size=block_size, rope_dim=0, reserved=rounding,
                             values=_ptr(values), packed=_ptr(packed), scales=_ptr(scales))
        self._core("FP8 pack", self.lib.ferrule_hip_core_quantize_launch, a)
        return packed, scales

    def pack_fp4_rows_from_f32(self, values: torch.Tensor, block_size: int = 32,
                               rounding: int = abi.FP8_ROUND_CPU_REFERENCE):
        """f32 [rows, width] -> (e2m1 [rows, width/2], e8m0 [rows, width/block]); the
        reference's ``fp4_e2m1_e8m0_quantize_f32_packed`` (kernels.rs, kind 4)."""
        if values.dtype != torch.float32 or values.dim() != 2 or not values.is_contiguous():
            raise ValueError("pack_fp4_rows_from_f32 expects contiguous f32 [rows, width]")
        rows, width = values.shape
        if width % block_size or block_size % 2:
            raise ValueError(f"row width {width} is not a multiple of block {block_size}")
        packed = torch.empty((rows, width // 2), dtype=torch.uint8, device=self.device)
        scales = torch.empty((rows, width // block_size), dtype=torch.uint8, device=self.device)
        a = abi.QuantizeArgs(kind=abi.QUANTIZE_FP4_PACKED, value_offset=0, value_len=rows * width,
                             row_width=width, block_size=block_size, rope_dim=0, reserved=rounding,
                             values=_ptr(values), packed=_ptr(packed), scales=_ptr(scales))
        self._core("FP4 pack", self.lib.ferrule_hip_core_quantize_launch, a)
        return packed, scales

    def artifact_linear_matvec_into(self, handle: HipArtifactLinearHandle, x: torch.Tensor,
                                    out: torch.Tensor, quantize_input: bool = False) -> torch.Tensor:
        """f32 activations -> f32 outputs for an FP8/E8M0 artifact (context.rs:5726-5759:
        kind 8 when the caller wants the K-block activation quantization, else kind 4)."""
        sh = handle.shape
        if sh.weight_format != abi.WEIGHT_FP8_E4M3 or sh.scale_kind != abi.SCALE_E8M0:
            raise ProviderError("artifact_linear_matvec_into (FP8/E8M0 artifacts only)", abi.UNSUPPORTED)
        if x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] != sh.in_features or not x.is_contiguous():
            raise ValueError("linear input must be contiguous f32 [batch, in_features]")
        if out.dtype != torch.float32 or tuple(out.shape) != (x.shape[0], sh.out_features):
            raise ValueError("linear output must be f32 [batch, out_features]")
        kind = abi.LINEAR_FP8_E4M3_E8M0_FROM_F32 if quantize_input else abi.LINEAR_FP8_E4M3_E8M0
        a = abi.LinearArgs(kind=kind, batch=x.shape[0], n=sh.out_features, k=sh.in_features,
                           scale_cols=sh.scale_cols, block_m=sh.block_m, block_k=sh.block_k,
                           x=_ptr(x), x_scales=0, weight=_ptr(handle.weight),
                           weight_scales=_ptr(handle.scale), output=_ptr(out))
        self._core("linear", self.lib.ferrule_hip_core_linear_launch, a)
        return out

    def gemm_fp8_e4m3fn_e8m0_prepacked(self, handle: HipArtifactLinearHandle, x_packed: torch.Tensor,
                                       x_scales: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """e4m3 activations + per-K128 e8m0 scales -> f32 (kind 5; the reference's
        ``gemm_fp8_e4m3fn_e8m0_prepacked``, context.rs:10766-10785)."""
        sh = handle.shape
        a = abi.LinearArgs(kind=abi.LINEAR_FP8_E4M3_E8M0_PACKED, batch=x_packed.shape[0], n=sh.out_features,
                           k=sh.in_features, scale_cols=sh.in_features // 128, block_m=128, block_k=128,
                           x=_ptr(x_packed), x_scales=_ptr(x_scales), weight=_ptr(handle.weight),
                           weight_scales=_ptr(handle.scale), output=_ptr(out))
        self._core("prepacked linear", self.lib.ferrule_hip_core_linear_launch, a)
        return out

    def synchronize(self) -> None:
        self.stream.synchronize()
