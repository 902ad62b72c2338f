"""Host mirror of the reference's projection seams, issuing HIP kernels through the C ABI.

``QuantizedProjections`` mirrors J/backend/tornado/layers/QuantizedProjections.java (decode, one
activation vector) and ``QuantizedBatchProjections`` mirrors
J/backend/tornado/layers/QuantizedBatchProjections.java (``batchSize`` activation rows), with the
same method names, argument meaning (``n`` = row length, ``d`` = output rows) and error behaviour:
a combination with no kernel raises, it never runs something else.  Where the reference adds a task
to a TaskGraph, these enqueue the kernel on the context's stream; the ``graph`` / ``name`` arguments
of the reference therefore disappear.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

from . import _lib as L
from .ggml import GGMLType
from .runtime import Context, DeviceBuffer, FloatArray, HalfFloatArray, ResidentCopies, TornadoTensor

# QuantizedProjections.fusedGateUp (:386-393): Q8_0, Q4_0, Q4_K and Q5_K;
# QuantizedBatchProjections.fusedGateUp (:315-321), the tiled answer: Q8_0, Q4_0 and Q4_K
FUSED_GATE_UP_TYPES = (GGMLType.Q8_0, GGMLType.Q4_0, GGMLType.Q4_K, GGMLType.Q5_K)
BATCH_FUSED_GATE_UP_TYPES = (GGMLType.Q8_0, GGMLType.Q4_0, GGMLType.Q4_K)


@dataclass
class TornadoWorkspace:
    """The persistent activation arrays a layer's projections read and write
    (J/backend/tornado/workspace/TornadoWorkspace.java): bound once, values move, arrays never."""
    wrapX: FloatArray | None = None
    wrapXb: FloatArray | None = None
    wrapHb: FloatArray | None = None
    wrapHb2: FloatArray | None = None
    # the packed-integer path's view of the current activation (PackedActivationTasks' arrays)
    packedX: "PackedActivation | None" = None


class PackedActivation:
    """An activation vector as Q8 blocks on the device: ``n`` signed bytes, ``n / 32`` fp32 scales
    and ``n / 32`` int32 block sums (quantizeActivationQ8Blocks,
    J/backend/tornado/kernels/TransformerComputeKernelsQ4_0.java:287-341)."""

    def __init__(self, context: Context, n: int):
        if n % 32:
            raise ValueError(f"{n} activations are not a whole number of blocks of 32")
        self.n = n
        self.quants = context.raw_buffer(n)
        self.scales = context.raw_buffer(n // 32 * 4)
        self.sums = context.raw_buffer(n // 32 * 4)

    def get(self):
        """(int8 quants, float32 scales, int32 sums) on the host."""
        import numpy as np
        return (self.quants.download(np.int8, self.n), self.scales.download(np.float32, self.n // 32),
                self.sums.download(np.int32, self.n // 32))


def _check_shape(w: TornadoTensor, n: int, d: int) -> None:
    if (w.cols, w.rows) != (n, d):
        raise ValueError(f"weight is {w.rows}x{w.cols}, projection asked for d={d}, n={n}")


class QuantizedProjections:
    """Single-token projections over weights kept in the file's representations."""

    def __init__(self, context: Context, ws: TornadoWorkspace, packed: bool = False):
        self.context = context
        self.ws = ws
        self._lib = context._lib
        self._packed = packed

    def packed(self) -> bool:
        """Whether the projections take the packed-integer path (QuantizedProjections.java:110-112):
        one answer for the whole layer, faster and looser -- the activation keeps 8 bits.  Off unless
        asked for; the fp32 path is the one held to the CPU path's results."""
        return self._packed

    def quantize(self, x: FloatArray, n: int) -> None:
        """``ws.packedX`` = ``x`` as Q8 blocks (PackedActivationTasks.quantize,
        QuantizedProjections.java:296-298)."""
        px = self.ws.packedX
        if px is None or px.n != n:
            raise RuntimeError("the packed path needs ws.packedX bound to a PackedActivation of the row length")
        L.check(self._lib.jl_quantize_q8(self.context.handle, x.ptr, n, px.quants.ptr, px.scales.ptr, px.sums.ptr))

    def rmsApply(self, rmsWeights: FloatArray, temp: FloatArray, n: int) -> None:
        """``wrapXb = rmsWeights * (temp[0] * wrapX)``, quantised as well where the projections are
        packed (QuantizedProjections.rmsApply, QuantizedProjections.java:117-130: reductionOneBlock2WithLayer,
        or PackedActivationTasks.rmsApplyAndQuantize).  ``temp`` is the scalar ``rmsScale`` leaves."""
        if self.packed():
            self.rmsApplyAndQuantize(self.ws.wrapX, rmsWeights, temp, n)
            return
        L.check(self._lib.jl_rms_apply(self.context.handle, self.ws.wrapX.ptr, rmsWeights.ptr, temp.ptr, n,
                                       self.ws.wrapXb.ptr))

    def rmsApplyAndQuantize(self, x: FloatArray, rmsWeights: FloatArray, rmsScale: FloatArray, n: int) -> None:
        """``wrapXb = rmsWeights * (rmsScale[0] * x)`` and ``packedX`` = its Q8 blocks, in one launch
        (QuantizedProjections.rmsApply, QuantizedProjections.java:117-121 ->
        PackedActivationTasks.rmsApplyAndQuantize)."""
        px = self.ws.packedX
        if px is None or px.n != n:
            raise RuntimeError("the packed path needs ws.packedX bound to a PackedActivation of the row length")
        L.check(self._lib.jl_rms_quantize_q8(self.context.handle, x.ptr, rmsWeights.ptr, rmsScale.ptr, n,
                                             self.ws.wrapXb.ptr, px.quants.ptr, px.scales.ptr, px.sums.ptr))

    def packedMatvec(self, out: FloatArray, w: TornadoTensor, n: int, d: int, residual: bool = False) -> None:
        """``out (+)= w . packedX`` (the packed arms of QuantizedProjections.java:156-190, 299-346)."""
        _check_shape(w, n, d)
        px = self.ws.packedX
        L.check(self._lib.jl_gemv_q8(self.context.handle, w.handle, px.quants.ptr, px.scales.ptr, px.sums.ptr,
                                     out.ptr, L.JL_RESIDUAL if residual else L.JL_STORE))

    def packedFusedQKV(self, q: FloatArray, k: FloatArray, v: FloatArray, wq: TornadoTensor, wk: TornadoTensor,
                       wv: TornadoTensor) -> None:
        """fusedQKVMatmulQ8_0DP4A and its siblings over ``packedX``."""
        px = self.ws.packedX
        L.check(self._lib.jl_gemv_qkv_q8(self.context.handle, wq.handle, wk.handle, wv.handle, px.quants.ptr,
                                         px.scales.ptr, px.sums.ptr, q.ptr, k.ptr, v.ptr))

    def packedGateUp(self, w1: TornadoTensor, w3: TornadoTensor, n: int, d: int) -> None:
        """``wrapHb = SiLU(w1 . packedX) * (w3 . packedX)`` (fusedFFNGateUpSiLUQ8_0DP4A and siblings)."""
        _check_shape(w1, n, d)
        _check_shape(w3, n, d)
        px = self.ws.packedX
        L.check(self._lib.jl_gemv_gate_up_q8(self.context.handle, w1.handle, w3.handle, px.quants.ptr,
                                             px.scales.ptr, px.sums.ptr, self.ws.wrapHb.ptr))

    def matvec(self, out: FloatArray, w: TornadoTensor, n: int, d: int) -> None:
        """``out = w . wrapXb`` (QuantizedProjections.java:140-194)."""
        self.floatMatvec(self.ws.wrapXb, out, w, n, d)

    def floatMatvec(self, x: FloatArray, out: FloatArray, w: TornadoTensor, n: int, d: int) -> None:
        """``out = w . x`` (QuantizedProjections.java:200-254)."""
        _check_shape(w, n, d)
        L.check(self._lib.jl_gemv(self.context.handle, w.handle, x.ptr, out.ptr, L.JL_STORE))

    def residualMatvec(self, x: FloatArray, w: TornadoTensor, n: int, d: int) -> None:
        """``wrapX += w . x`` (QuantizedProjections.java:260-379)."""
        _check_shape(w, n, d)
        L.check(self._lib.jl_gemv(self.context.handle, w.handle, x.ptr, self.ws.wrapX.ptr,
                                  L.JL_RESIDUAL))

    def fusedQKV(self, x: FloatArray, q: FloatArray, k: FloatArray, v: FloatArray,
                 wq: TornadoTensor, wk: TornadoTensor, wv: TornadoTensor) -> None:
        """q | k | v in one launch (fusedQKVMatmulQ8 and its Q4_0 / Q4_K siblings, called directly
        on the kernels by the reference's layer builders, LlamaQ8_0FFNLayers.java:316-329)."""
        L.check(self._lib.jl_gemv_qkv(self.context.handle, wq.handle, wk.handle, wv.handle, x.ptr,
                                      q.ptr, k.ptr, v.ptr))

    def fusedGateUp(self, w1: TornadoTensor, w3: TornadoTensor) -> bool:
        """QuantizedProjections.java:386-393."""
        return w1.data_type() == w3.data_type() and w1.data_type() in FUSED_GATE_UP_TYPES

    def gateUp(self, w1: TornadoTensor, w3: TornadoTensor, n: int, d: int) -> None:
        """``wrapHb = SiLU(w1 . wrapXb) * (w3 . wrapXb)`` (QuantizedProjections.java:400-480): one
        fused launch where both weights share a type, else two projections into ``wrapHb`` and
        ``wrapHb2`` and an element-wise SwiGLU."""
        _check_shape(w1, n, d)
        _check_shape(w3, n, d)
        if self.fusedGateUp(w1, w3):
            L.check(self._lib.jl_gemv_gate_up(self.context.handle, w1.handle, w3.handle,
                                              self.ws.wrapXb.ptr, self.ws.wrapHb.ptr))
            return
        if self.ws.wrapHb2 is None:
            raise RuntimeError("a layer that splits gate and up needs wrapHb2 bound")
        self.matvec(self.ws.wrapHb, w1, n, d)
        self.matvec(self.ws.wrapHb2, w3, n, d)
        L.check(self._lib.jl_swiglu(self.context.handle, self.ws.wrapHb.ptr, self.ws.wrapHb2.ptr, d))


    # ---- the reference's fused decode kernels: RMS normalisation folded into the projection ----

    def rmsScale(self, x: FloatArray, n: int, eps: float, scale: FloatArray) -> None:
        """``scale[0] = 1 / sqrt(sum x^2 / n + eps)`` on the device (reductionOneBlockWithLayer,
        TransformerComputeKernels.java:378-437; CpuOperations.rmsnorm :60-66)."""
        L.check(self._lib.jl_rms_scale(self.context.handle, x.ptr, n, float(eps), scale.ptr))

    def rmsMatvec(self, x: FloatArray, rmsWeights: FloatArray, rmsScale: FloatArray | None,
                  out: FloatArray, w: TornadoTensor, n: int, d: int, eps: float = 0.0) -> None:
        """``out = w . (rmsWeights * (s * x))``: the final norm folded into the vocabulary
        projection (reductionOneBlock2WithLogits + the projection, LogitsQ8_0Layer.java:85-97).
        ``s`` is ``rmsScale[0]``, or with ``rmsScale`` None computed in the kernel from ``eps``."""
        _check_shape(w, n, d)
        L.check(self._lib.jl_gemv_rms(self.context.handle, w.handle, x.ptr, rmsWeights.ptr,
                                      rmsScale.ptr if rmsScale is not None else None, float(eps),
                                      out.ptr, L.JL_STORE))

    def fusedRmsNormQKV(self, x: FloatArray, q: FloatArray, k: FloatArray, v: FloatArray,
                        rmsWeights: FloatArray, rmsScale: FloatArray | None, wq: TornadoTensor,
                        wk: TornadoTensor, wv: TornadoTensor, eps: float = 0.0) -> None:
        """fusedRmsNormQKVMatmulQ8 (TransformerComputeKernelsLayered.java:2116-2220): q | k | v of
        the normalised activations, which are never written out.  With ``rmsScale`` None the scale
        is computed in the kernel from ``eps`` and the separate reduction is not needed."""
        L.check(self._lib.jl_gemv_qkv_rms(self.context.handle, wq.handle, wk.handle, wv.handle, x.ptr,
                                          rmsWeights.ptr,
                                          rmsScale.ptr if rmsScale is not None else None, float(eps),
                                          q.ptr, k.ptr, v.ptr))

    def fullyFusedRmsNormGateUp(self, x: FloatArray, rmsWeights: FloatArray, eps: float,
                                w1: TornadoTensor, w3: TornadoTensor, n: int, d: int) -> None:
        """fullyFusedRmsNormFFNGateUpQ8 (TransformerComputeKernelsLayered.java:2866+):
        ``wrapHb = SiLU(w1 . xn) * (w3 . xn)`` with ``xn`` the RMS-normalised ``x``, the scale
        computed inside the kernel."""
        _check_shape(w1, n, d)
        _check_shape(w3, n, d)
        L.check(self._lib.jl_gemv_gate_up_rms(self.context.handle, w1.handle, w3.handle, x.ptr,
                                              rmsWeights.ptr, float(eps), self.ws.wrapHb.ptr))

    def argmax(self, logits: FloatArray, n: int, token: DeviceBuffer) -> None:
        """``token[0]`` = index of the first maximum of the logits, an int32 on the device
        (argmaxLogits, TransformerComputeKernels.java:95-127)."""
        L.check(self._lib.jl_argmax(self.context.handle, logits.ptr, n, token.ptr))


    def matvecArgmax(self, x: FloatArray, logits: FloatArray, w: TornadoTensor, n: int, d: int,
                     token: DeviceBuffer, rmsWeights: FloatArray | None = None,
                     rmsScale: FloatArray | None = None, eps: float = 0.0) -> None:
        """The tail of a greedy decode step in one call: ``logits = w . x`` -- with ``rmsWeights`` set,
        of the RMS-normalised ``x`` as in ``rmsMatvec`` -- and ``token[0]`` = ``argmax(logits)``
        (the vocabulary projection followed by "argmax_sample", LogitsQ8_0Layer.java:92-110).  Bit for
        bit what ``matvec`` / ``rmsMatvec`` followed by ``argmax`` leave; where the projection kernel
        can keep its workgroups' best logits, one launch fewer."""
        _check_shape(w, n, d)
        L.check(self._lib.jl_gemv_argmax(self.context.handle, w.handle, x.ptr,
                                         rmsWeights.ptr if rmsWeights is not None else None,
                                         rmsScale.ptr if rmsScale is not None else None, float(eps),
                                         logits.ptr, token.ptr))


class QuantizedBatchProjections:
    """Projections of ``batchSize`` activation rows at once (batched decode, batched prefill)."""

    def __init__(self, context: Context, batchSize: int, max_cols: int, max_out_cols: int = 0,
                 math: int = L.JL_MATH_DEFAULT, resident: bool = False):
        """``max_cols`` is the longest row any projection reads, ``max_out_cols`` the most output
        columns one call produces (gate + up rows for a fused gate/up); together they size the
        workspace once, before anything runs (Implementation.needs)."""
        self.context = context
        self.batchSize = int(batchSize)
        self.math = math
        self._lib = context._lib
        self._max_cols = int(max_cols)
        nbytes = self._lib.jl_gemm_workspace_bytes(self.batchSize, self._max_cols, int(max_out_cols), math)
        self.workspace = DeviceBuffer(context, max(nbytes, 256))
        # the reference's residency choice for the batched prefill (BatchPrefillWorkspace;
        # dequantize*ToFP16Once): an fp16 copy per set of weights that outlives the call
        self.resident = bool(resident)
        self._copies = ResidentCopies(context)

    def workspace_bytes(self) -> int:
        return self.workspace.nbytes

    def _gemm(self, weights, x: FloatArray, out: FloatArray, activeRows: int, ldo: int,
              colOffset: int, epilogue: int) -> None:
        n = weights[0].cols
        if n > self._max_cols:
            raise ValueError(f"row length {n} exceeds the {self._max_cols} the workspace was sized for")
        arr = (C.c_void_p * len(weights))(*[w.handle for w in weights])
        copy, state = None, None
        if self.resident:
            copy, state = self._copies.lookup(weights, epilogue == L.JL_SWIGLU,
                                              lambda: self._lib.jl_gemm_resident_bytes(arr, len(weights)))
        if isinstance(x, HalfFloatArray):
            # fp16 activations, the operand type of the reference's prefill GEMMs (gemmMMA's
            # HalfFloatArray A); an fp16 ``out`` is the hidden vector batchedFFNSwiGLUFP16Packed writes
            L.check(self._lib.jl_gemm_xf16(
                self.context.handle, arr, len(weights), x.ptr, out.ptr, int(isinstance(out, HalfFloatArray)),
                self.batchSize, activeRows, ldo, colOffset, epilogue, self.workspace.ptr, self.workspace.nbytes,
                copy.ptr if copy else None, copy.nbytes if copy else 0, C.byref(state) if copy else None))
            return
        if isinstance(out, HalfFloatArray):
            raise ValueError("an fp16 output needs fp16 activations")
        if not self.resident:
            L.check(self._lib.jl_gemm(self.context.handle, arr, len(weights), x.ptr, out.ptr,
                                      self.batchSize, activeRows, ldo, colOffset, epilogue, self.math,
                                      self.workspace.ptr, self.workspace.nbytes))
            return
        L.check(self._lib.jl_gemm_resident(self.context.handle, arr, len(weights), x.ptr, out.ptr,
                                           self.batchSize, activeRows, ldo, colOffset, epilogue, self.math,
                                           self.workspace.ptr, self.workspace.nbytes, copy.ptr, copy.nbytes,
                                           C.byref(state)))

    def rmsApplyFP16(self, x: FloatArray, rmsWeights: FloatArray, eps: float, out: HalfFloatArray, dim: int,
                     scales: FloatArray | None = None, activeRows: int | None = None,
                     delta: FloatArray | None = None) -> None:
        """``out[b] = fp16(rmsWeights * scale_b * x[b])`` with ``scale_b`` from the row's mean square:
        batchedRmsReduceParallel + batchedRmsApplyFP16 (TransformerBatchPrefillKernels.java:1480-1510,
        59-72), the step that hands the prefill projections their fp16 activations.  With ``delta``
        the pending residual add ``x += delta`` comes first (batchedRmsReduceFusedResidual, :1519-1551)."""
        rows = self.batchSize if activeRows is None else activeRows
        L.check(self._lib.jl_rms_apply_xf16(self.context.handle, x.ptr, delta.ptr if delta is not None else None,
                                            rmsWeights.ptr, eps, rows, dim,
                                            scales.ptr if scales is not None else None, out.ptr))

    def argmaxLogits(self, logits: FloatArray, vocab: int, tokens: DeviceBuffer, activeRows: int | None = None,
                     rowStride: int | None = None) -> None:
        """``tokens[b]`` = first maximum of row ``b`` of the batched logits, int32 on the device
        (batchedArgmaxLogits, TransformerBatchPrefillKernels.java:2118-2159; the "argmax" task of
        TornadoBatchExecutor's logits graph, :226-232): only the batch's token ids go to the host."""
        rows = self.batchSize if activeRows is None else activeRows
        L.check(self._lib.jl_argmax_rows(self.context.handle, logits.ptr, rows, vocab,
                                         vocab if rowStride is None else rowStride, tokens.ptr))

    def projection(self, x: FloatArray, out: FloatArray, w: TornadoTensor, n: int, d: int,
                   residual: bool, activeRows: int | None = None) -> None:
        """``out = w . x`` over the batch, or ``out += w . x`` with ``residual``
        (QuantizedBatchProjections.java:76-309).  Rows past ``activeRows`` are left untouched."""
        _check_shape(w, n, d)
        rows = self.batchSize if activeRows is None else activeRows
        self._gemm([w], x, out, rows, d, 0, L.JL_RESIDUAL if residual else L.JL_STORE)

    def fusedQKV(self, x: FloatArray, out: FloatArray, wq: TornadoTensor, wk: TornadoTensor,
                 wv: TornadoTensor, activeRows: int | None = None) -> None:
        """``out[b] = [wq . x_b | wk . x_b | wv . x_b]``, the side-by-side layout of the
        reference's FP16Projections (C = A . [W0|W1|W2]^T)."""
        rows = self.batchSize if activeRows is None else activeRows
        ldo = wq.rows + wk.rows + wv.rows
        self._gemm([wq, wk, wv], x, out, rows, ldo, 0, L.JL_STORE)

    def fusedGateUp(self, w1: TornadoTensor, w3: TornadoTensor) -> bool:
        """QuantizedBatchProjections.java:315-321 (the tiled, non-SIMD-group answer)."""
        return w1.data_type() == w3.data_type() and w1.data_type() in BATCH_FUSED_GATE_UP_TYPES

    def gateUp(self, x: FloatArray, hb: FloatArray, w1: TornadoTensor, w3: TornadoTensor, dim: int,
               hidDim: int, activeRows: int | None = None) -> None:
        """``hb = SiLU(w1 . x) * (w3 . x)`` over the batch, for every pair of weight types
        (QuantizedBatchProjections.java:329-458;
        the RMS norm the reference folds in front is not part of this path: ``x`` is already
        normalised)."""
        _check_shape(w1, dim, hidDim)
        _check_shape(w3, dim, hidDim)
        # Where fusedGateUp does not hold the reference runs gate into wrapHbBatch, up into
        # ffnUpResult and siluAndMultiply (:446-457); jl_gemm takes any pair of types the library
        # decodes -- equal or not -- with the SwiGLU as its epilogue, so it is one call either way.
        rows = self.batchSize if activeRows is None else activeRows
        self._gemm([w1, w3], x, hb, rows, hidDim, 0, L.JL_SWIGLU)
