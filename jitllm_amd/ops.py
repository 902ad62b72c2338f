"""Host mirror of the reference's batched-prefill plugin seam, with the HIP library behind it.

The reference chooses, step by step, the first *implementation* of an ordered candidate list whose
fusion table matches the next operations and that accepts the step
(J/backend/tornado/ops/WorkPlan.java:36-68, Implementations.java:19-26; J = src/main/java/org/
beehive/jitllm).  This module restates the types that choice is made of -- ``OperationKind``,
``MatMul``, ``SwiGLU``, ``ResidualAdd``, ``Fusion``, ``Step``, ``Target``,
``BatchPrefillWorkspace``, ``Implementation``, ``Instance`` -- with the reference's names, argument
meaning and error behaviour, and adds the candidate a maintainer would list first:
``HipImplementation`` (``library() == "hip"``), whose ``Instance`` runs the steps through
``jl_gemm`` / ``jl_gemm_resident``.  Where the reference's ``emit`` adds tasks to a TaskGraph, this
one enqueues the kernels on the context's stream, as the other mirrors in this package do.
"""
from __future__ import annotations

import ctypes as C
import enum
import os
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

from . import _lib as L
from .ggml import GGMLType
from .runtime import Context, DeviceBuffer, FloatArray, HalfFloatArray, ResidentCopies, TornadoTensor


class OperationKind(enum.Enum):
    """The kinds this path meets (J/program/op/OperationKind.java:15-60)."""
    RMS_NORM = "RMS_NORM"
    MAT_MUL = "MAT_MUL"
    SWIGLU = "SWIGLU"
    RESIDUAL_ADD = "RESIDUAL_ADD"


class TensorRole(enum.Enum):
    ATTENTION_QUERY = "ATTENTION_QUERY"
    ATTENTION_KEY = "ATTENTION_KEY"
    ATTENTION_VALUE = "ATTENTION_VALUE"
    ATTENTION_OUTPUT = "ATTENTION_OUTPUT"
    FFN_GATE = "FFN_GATE"
    FFN_UP = "FFN_UP"
    FFN_DOWN = "FFN_DOWN"
    ATTENTION_NORM = "ATTENTION_NORM"
    FFN_NORM = "FFN_NORM"


@dataclass(frozen=True)
class MatMul:
    """A weight matrix times a batch of activation rows (J/program/op/MatMul.java:22-46): ``weight``
    is the role of the layer's weight, ``input`` / ``output`` are activation names."""
    weight: TensorRole
    input: str
    output: str
    rows: int
    columns: int
    batchSize: int
    dataType: GGMLType
    kind = OperationKind.MAT_MUL

    def __post_init__(self):
        if self.rows <= 0 or self.columns <= 0:
            raise ValueError(f"rows and columns must be positive: {self.rows}x{self.columns}")
        if self.batchSize <= 0:
            raise ValueError(f"batchSize must be positive: {self.batchSize}")


@dataclass(frozen=True)
class SwiGLU:
    """``output = SiLU(gate) * up`` (J/program/op/SwiGLU.java)."""
    gate: str
    up: str
    output: str
    kind = OperationKind.SWIGLU


@dataclass(frozen=True)
class ResidualAdd:
    """``residual += input`` (J/program/op/ResidualAdd.java)."""
    residual: str
    input: str
    kind = OperationKind.RESIDUAL_ADD


@dataclass(frozen=True)
class RmsNorm:
    """``output = input / rms(input) * weight`` over rows of ``groupLength`` values
    (J/program/op/RmsNorm.java:44-60).  ``weight`` is the role of the learned scale, None for the
    unweighted form; ``groups`` above 1 is the per-head form."""
    input: str
    output: str
    weight: Optional[TensorRole] = None
    epsilon: float = 1e-5
    groupLength: int = 0
    groups: int = 1
    kind = OperationKind.RMS_NORM

    def __post_init__(self):
        if self.groups < 1:
            raise ValueError(f"groups must be at least 1: {self.groups}")
        if self.groups > 1 and self.groupLength < 1:
            raise ValueError(f"a norm over {self.groups} groups must state the group length")


@dataclass(frozen=True)
class Fusion:
    """A sequence of operation kinds an implementation runs as one step, with an extra condition
    on the matched operations (J/backend/tornado/ops/Fusion.java:17-58)."""
    name: str
    kinds: tuple
    check: Callable[[Sequence], bool] = field(default=lambda ops: True, compare=False)

    def __post_init__(self):
        if not self.kinds:
            raise ValueError("a fusion needs at least one operation")

    @staticmethod
    def of(name: str, *kinds: OperationKind) -> "Fusion":
        return Fusion(name, tuple(kinds))

    def when(self, condition: Callable[[Sequence], bool]) -> "Fusion":
        prior = self.check
        return Fusion(self.name, self.kinds, lambda ops: prior(ops) and condition(ops))

    def match(self, ops: Sequence, at: int) -> Optional[list]:
        if at + len(self.kinds) > len(ops):
            return None
        candidate = list(ops[at:at + len(self.kinds)])
        for op, kind in zip(candidate, self.kinds):
            if op.kind != kind:
                return None
        return candidate if self.check(candidate) else None

    @staticmethod
    def sameInput(ops: Sequence) -> bool:
        """Whether every projection in ``ops`` reads the same input, as q, k and v do."""
        inputs = {op.input for op in ops if isinstance(op, MatMul)}
        return len(inputs) <= 1


# The tensor-core fusion table (J/backend/tornado/ops/TensorCoreSteps.java:44-78), longest first.
QKV = Fusion.of("q|k|v", OperationKind.MAT_MUL, OperationKind.MAT_MUL, OperationKind.MAT_MUL).when(Fusion.sameInput)
GATE_UP_SWIGLU = Fusion.of("gate|up + SwiGLU", OperationKind.MAT_MUL, OperationKind.MAT_MUL,
                           OperationKind.SWIGLU).when(Fusion.sameInput)
DOWN_ADD = Fusion.of("down + residual add", OperationKind.MAT_MUL, OperationKind.RESIDUAL_ADD).when(
    lambda ops: ops[0].weight == TensorRole.FFN_DOWN)
GATE_UP = Fusion.of("gate|up", OperationKind.MAT_MUL, OperationKind.MAT_MUL).when(Fusion.sameInput).when(
    lambda ops: ops[0].weight == TensorRole.FFN_GATE and ops[1].weight == TensorRole.FFN_UP)
PROJECTION = Fusion.of("projection", OperationKind.MAT_MUL)
ADD_NORM = Fusion.of("residual add + RMS norm", OperationKind.RESIDUAL_ADD, OperationKind.RMS_NORM)
NORM = Fusion.of("RMS norm", OperationKind.RMS_NORM)
RESIDUAL = Fusion.of("residual add", OperationKind.RESIDUAL_ADD)
FUSIONS = [QKV, GATE_UP_SWIGLU, ADD_NORM, DOWN_ADD, GATE_UP, PROJECTION, NORM, RESIDUAL]


def scaleOf(norm: RmsNorm) -> str:
    """The name of a norm's row-scale buffer: its output's name and ".scale" (TensorCoreSteps.java:291-294)."""
    return norm.output + ".scale"


@dataclass(frozen=True)
class Step:
    """Operations of one layer that one implementation runs together
    (J/backend/tornado/ops/Step.java:17-62)."""
    layer: int
    tokens: int
    fusion: Fusion
    ops: tuple

    def matMuls(self) -> List[MatMul]:
        return [op for op in self.ops if isinstance(op, MatMul)]

    def first(self, kind: type):
        for op in self.ops:
            if isinstance(op, kind):
                return op
        raise ValueError(f"{self.fusion.name} has no {kind.__name__}")

    def weights(self) -> int:
        return sum(m.rows * m.columns for m in self.matMuls())

    def outputWidth(self) -> int:
        return sum(m.rows for m in self.matMuls())


@dataclass(frozen=True)
class Target:
    """What an implementation is chosen for: the session's options and what the device can do
    (J/backend/tornado/ops/Target.java:12-35)."""
    nativeLibraries: bool = True
    capabilities: frozenset = frozenset({"TENSOR_CORE_MMA"})

    def supports(self, capability: str) -> bool:
        return capability in self.capabilities

    def hip(self) -> bool:
        """The analogue of ``Target.cublas()``: native libraries allowed, matrix cores, and the
        library loads (a missing library is 'loads -> false', never an exception:
        LibraryProbe)."""
        if not (self.nativeLibraries and self.supports("TENSOR_CORE_MMA")):
            return False
        try:
            L.load()
        except (OSError, FileNotFoundError, AttributeError):
            return False
        return True


@dataclass(frozen=True)
class BatchPrefillWorkspace:
    """Device bytes ``create`` will allocate, computed up front so that the memory preflight equals
    the allocation (J/backend/tornado/ops/Implementation.java:31-36, WorkPlan.java:18-21):
    ``bytes`` always, ``residentBytes`` on top when the plan chooses residency."""
    bytes: int
    residentBytes: int = 0

    @staticmethod
    def withoutResidencyChoice(n: int) -> "BatchPrefillWorkspace":
        return BatchPrefillWorkspace(int(n), 0)


class Operands:
    """The arrays behind the names the operations use (J/backend/tornado/ops/Operands.java:17-33)."""

    def __init__(self, activations: Dict[str, FloatArray],
                 weights: Callable[[TensorRole, int], TornadoTensor]):
        self._activations = dict(activations)
        self._weights = weights

    def activation(self, name: str) -> FloatArray:
        if name not in self._activations:
            raise ValueError(f"no array for activation {name}")
        return self._activations[name]

    def weight(self, role: TensorRole, layer: int) -> TornadoTensor:
        return self._weights(role, layer)


class Instance:
    """An implementation after allocation (J/backend/tornado/ops/Instance.java:8-23)."""

    def buffers(self) -> list:
        return []

    def emit(self, step: Step, operands: Operands) -> None:
        raise NotImplementedError

    def addGrids(self, scheduler=None) -> None:
        """The library's launches carry their own grids."""


class Implementation:
    """One way to run program operations (J/backend/tornado/ops/Implementation.java:16-49)."""

    def library(self) -> str:
        return "none"

    def fusions(self) -> List[Fusion]:
        raise NotImplementedError

    def accepts(self, step: Step, target: Target) -> bool:
        raise NotImplementedError

    def needs(self, steps: Sequence[Step], target: Target) -> BatchPrefillWorkspace:
        return BatchPrefillWorkspace.withoutResidencyChoice(0)

    def create(self, steps: Sequence[Step], target: Target, context: Context, prepacking=None) -> Instance:
        raise NotImplementedError

    def narrowed(self, primary: Instance, steps: Sequence[Step], target: Target, context: Context,
                 prepacking=None) -> Instance:
        return self.create(steps, target, context, prepacking)


SUPPORTED = frozenset(GGMLType)


def _sizes(steps: Sequence[Step]):
    rows = max(s.tokens for s in steps)
    cols = max(m.columns for s in steps for m in s.matMuls())
    widest = max(s.outputWidth() for s in steps)
    return rows, cols, widest


class HipImplementation(Implementation):
    """The batched prefill through libjitllm_hip.so.  Listed ahead of the JIT candidates it claims
    the projection steps whose weights it has kernels for; everything else falls through."""

    def __init__(self, residency: bool = False, splitK: Optional[bool] = None):
        self.residency = bool(residency)
        # -Djitllm.prefill.splitK=false keeps every GEMM whole (SplitKGemm.java:40-42); here the
        # environment variable JITLLM_PREFILL_SPLITK=false, unless the caller says
        if splitK is None:
            splitK = os.environ.get("JITLLM_PREFILL_SPLITK", "true").lower() != "false"
        self.splitK = bool(splitK)

    def library(self) -> str:
        return "hip"

    def fusions(self) -> List[Fusion]:
        return list(FUSIONS)

    def accepts(self, step: Step, target: Target) -> bool:
        if not target.hip():
            return False
        mm = step.matMuls()
        name = step.fusion.name
        if name in (NORM.name, ADD_NORM.name):
            # the norm that feeds a GEMM its fp16 rows: one group over the row, a learned scale
            norm = step.first(RmsNorm)
            if norm.weight is None or norm.groups != 1 or norm.groupLength <= 0:
                return False
            return name == NORM.name or step.first(ResidualAdd).residual == norm.input
        if name == RESIDUAL.name:
            return True
        if not mm or len(mm) > 8:
            return False
        if any(m.dataType not in SUPPORTED for m in mm):
            return False
        # one call multiplies weights of one row length; their types may differ -- each is decoded
        # by its own, as tensorCoresOverDecoded asks only that every type be decodable
        # (DequantizingMatMul.java:53-63)
        if len({m.columns for m in mm}) != 1:
            return False
        if mm[0].columns % 64:
            return False
        if step.fusion.name == GATE_UP_SWIGLU.name and mm[0].rows != mm[1].rows:
            return False
        return True

    def needs(self, steps: Sequence[Step], target: Target) -> BatchPrefillWorkspace:
        steps = [s for s in steps if s.matMuls()]      # the norms and adds need no scratch
        if not steps:
            return BatchPrefillWorkspace.withoutResidencyChoice(0)
        rows, cols, widest = _sizes(steps)
        lib = L.load()
        nbytes = lib.jl_gemm_workspace_bytes(rows, cols, widest, L.JL_MATH_DEFAULT)
        resident = 0
        if self.residency:
            # 2 bytes per weight, rows padded to whole 256-row tiles (jl_gemm_resident_bytes)
            resident = sum((s.outputWidth() + 511) // 256 * 256 * s.matMuls()[0].columns * 2 for s in steps)
        return BatchPrefillWorkspace(int(nbytes), int(resident))

    def create(self, steps: Sequence[Step], target: Target, context: Context, prepacking=None) -> Instance:
        if prepacking is not None:
            raise RuntimeError("the hip implementation reads the file's blocks, not prepacked tiles")
        need = self.needs(steps, target)
        if not steps:
            raise ValueError("an instance runs at least one step")
        context.set_split_k(self.splitK)
        return HipInstance(context, max(s.tokens for s in steps), DeviceBuffer(context, max(need.bytes, 256)),
                           self.residency, ResidentCopies(context))

    def narrowed(self, primary: Instance, steps: Sequence[Step], target: Target, context: Context,
                 prepacking=None) -> Instance:
        """The narrow family shares the primary's buffers (Implementation.java:41-48)."""
        assert isinstance(primary, HipInstance)
        return HipInstance(context, primary.batchSize, primary.workspace, primary.residency, primary.copies)


class HipInstance(Instance):
    def __init__(self, context: Context, batchSize: int, workspace: DeviceBuffer, residency: bool, copies: ResidentCopies):
        self.context = context
        self.batchSize = int(batchSize)
        self.workspace = workspace
        self.residency = residency
        self.copies = copies
        self._lib = context._lib
        self._producers: Dict[str, MatMul] = {}     # output name -> the projection that wrote it

    def buffers(self) -> list:
        return [self.workspace] + self.copies.buffers()

    def emit(self, step: Step, operands: Operands) -> None:
        """One ``jl_gemm`` per step: q|k|v and gate|up write side by side into the first output's
        array (the reference's packed rows, DecodedMatMul.java:93-109), gate|up + SwiGLU writes the
        SwiGLU's output, down + residual add accumulates into the residual."""
        mm = step.matMuls()
        name = step.fusion.name
        if step.tokens > self.batchSize:
            raise ValueError(f"a step of {step.tokens} tokens in an instance built for {self.batchSize}")
        if name in (NORM.name, ADD_NORM.name):
            # RMS norm into the fp16 input of the next GEMM, the row scales kept beside it; with a
            # residual add in front, the add runs inside the same launch (TensorCoreSteps.norm,
            # TensorCoreSteps.java:209-277: batchedRmsReduceParallel / batchedRmsReduceFusedResidual,
            # then batchedRmsApplyFP16 / batchedFFNRmsApplyFP16)
            norm = step.first(RmsNorm)
            delta = operands.activation(step.first(ResidualAdd).input) if name == ADD_NORM.name else None
            out = operands.activation(norm.output)
            if not isinstance(out, HalfFloatArray):
                raise ValueError(f"the norm's output {norm.output} is the next GEMM's fp16 input")
            L.check(self._lib.jl_rms_apply_xf16(
                self.context.handle, operands.activation(norm.input).ptr, delta.ptr if delta is not None else None,
                operands.weight(norm.weight, step.layer).ptr, norm.epsilon, step.tokens, norm.groupLength,
                operands.activation(scaleOf(norm)).ptr, out.ptr))
            return
        if name == RESIDUAL.name:
            # x += down on its own: it follows the down projection (TensorCoreSteps.java:145-153)
            add = step.first(ResidualAdd)
            down = self._producers.get(add.input)
            if down is None or down.weight != TensorRole.FFN_DOWN:
                raise ValueError(f"a residual add on its own follows the down projection, not {add.input}")
            L.check(self._lib.jl_residual_add(self.context.handle, operands.activation(add.residual).ptr,
                                              operands.activation(add.input).ptr, step.tokens * down.rows))
            return
        weights = [operands.weight(m.weight, step.layer) for m in mm]
        x = operands.activation(mm[0].input)
        self._producers[mm[0].output] = mm[0]
        if name == GATE_UP_SWIGLU.name:
            out, epilogue, ldo = operands.activation(step.first(SwiGLU).output), L.JL_SWIGLU, mm[0].rows
        elif name == DOWN_ADD.name:
            out, epilogue, ldo = operands.activation(step.first(ResidualAdd).residual), L.JL_RESIDUAL, mm[0].rows
        else:
            out, epilogue, ldo = operands.activation(mm[0].output), L.JL_STORE, step.outputWidth()
        arr = (C.c_void_p * len(weights))(*[w.handle for w in weights])
        copy, state = None, None
        if self.residency:
            copy, state = self.copies.lookup(weights, epilogue == L.JL_SWIGLU,
                                             lambda: self._lib.jl_gemm_resident_bytes(arr, len(weights)))
        if isinstance(x, HalfFloatArray):
            # the reference's own operand types: fp16 in (DecodedMatMul.java:100-109), fp32 out, or --
            # the feed-forward hidden vector -- fp16 out (batchedFFNSwiGLUFP16Packed)
            L.check(self._lib.jl_gemm_xf16(
                self.context.handle, arr, len(weights), x.ptr, out.ptr, int(isinstance(out, HalfFloatArray)),
                self.batchSize, step.tokens, ldo, 0, epilogue, self.workspace.ptr, self.workspace.nbytes,
                copy.ptr if copy else None, copy.nbytes if copy else 0, C.byref(state) if copy else None))
            return
        if isinstance(out, HalfFloatArray):
            raise ValueError("an fp16 output needs fp16 activations")
        args = (self.context.handle, arr, len(weights), x.ptr, out.ptr, self.batchSize, step.tokens, ldo, 0,
                epilogue, L.JL_MATH_DEFAULT, self.workspace.ptr, self.workspace.nbytes)
        if not self.residency:
            L.check(self._lib.jl_gemm(*args))
            return
        L.check(self._lib.jl_gemm_resident(*args, copy.ptr, copy.nbytes, C.byref(state)))


@dataclass(frozen=True)
class Chosen:
    implementation: Implementation
    step: Step


def split(ops: Sequence, layer: int, tokens: int, candidates: Sequence[Implementation], target: Target,
          region: str = "layer") -> List[Chosen]:
    """WorkPlan.split (J/backend/tornado/ops/WorkPlan.java:36-68): walks the operations, at each
    position takes the first candidate with a matching fusion (longest first) that accepts the
    step; an operation no candidate runs is an error that names it."""
    chosen: List[Chosen] = []
    at = 0
    while at < len(ops):
        nxt = None
        for implementation in candidates:
            for fusion in implementation.fusions():
                match = fusion.match(ops, at)
                if match is None:
                    continue
                step = Step(layer, tokens, fusion, tuple(match))
                if implementation.accepts(step, target):
                    nxt = Chosen(implementation, step)
                    break
            if nxt is not None:
                break
        if nxt is None:
            raise RuntimeError(f"no implementation runs {ops[at].kind.value} in layer {layer} ({region})")
        chosen.append(nxt)
        at += len(nxt.step.ops)
    return chosen
