"""The batched-prefill plugin seam (jitllm_amd/ops.py): fusion matching, the first-accepting-candidate
walk and the memory preflight, which need no GPU."""
import pytest

from jitllm_amd import _lib as L
from jitllm_amd import ops
from jitllm_amd.ggml import GGMLType
from jitllm_amd.ops import (ADD_NORM, DOWN_ADD, GATE_UP_SWIGLU, NORM, PROJECTION, QKV, RESIDUAL, HipImplementation, MatMul,
                            OperationKind, ResidualAdd, RmsNorm, Step, SwiGLU, Target, TensorRole)

DIM, KV, FFN, T = 2048, 512, 8192, 512


def llama_layer(t=GGMLType.Q8_0, dim=DIM, weighted=True):
    """The operations of one Llama layer around attention, in program order (``weighted`` false: the
    norms without a learned scale, which the library has no kernel for)."""
    R = TensorRole
    att, ffn = (R.ATTENTION_NORM, R.FFN_NORM) if weighted else (None, None)
    return [
        RmsNorm("x", "xb", att, 1e-5, dim),
        MatMul(R.ATTENTION_QUERY, "xb", "q", dim, dim, T, t),
        MatMul(R.ATTENTION_KEY, "xb", "k", KV, dim, T, t),
        MatMul(R.ATTENTION_VALUE, "xb", "v", KV, dim, T, t),
        MatMul(R.ATTENTION_OUTPUT, "att", "xb2", dim, dim, T, t),
        ResidualAdd("x", "xb2"),
        RmsNorm("x", "xb", ffn, 1e-5, dim),
        MatMul(R.FFN_GATE, "xb", "hb", FFN, dim, T, t),
        MatMul(R.FFN_UP, "xb", "hb2", FFN, dim, T, t),
        SwiGLU("hb", "hb2", "hb"),
        MatMul(R.FFN_DOWN, "hb", "xb2", dim, FFN, T, t),
        ResidualAdd("x", "xb2"),
    ]


class JitNorms(ops.Implementation):
    """Stands for the reference's JIT candidate: it takes what the library leaves."""

    def fusions(self):
        return [ops.Fusion.of("RMS norm", OperationKind.RMS_NORM), ops.Fusion.of("residual add", OperationKind.RESIDUAL_ADD),
                ops.Fusion.of("SwiGLU", OperationKind.SWIGLU), PROJECTION]

    def accepts(self, step, target):
        return True


def test_the_first_accepting_candidate_takes_each_step():
    chosen = ops.split(llama_layer(), 3, T, [HipImplementation(), JitNorms()], Target())
    got = [(c.implementation.library(), c.step.fusion.name) for c in chosen]
    # the reference's own split of a Llama layer: the residual add after attention is merged into
    # the next RMS norm (DecodedMatMul.java:31-35)
    assert got == [("hip", NORM.name), ("hip", QKV.name), ("hip", PROJECTION.name), ("hip", ADD_NORM.name),
                   ("hip", GATE_UP_SWIGLU.name), ("hip", DOWN_ADD.name)]
    # norms without a learned scale stay with the next candidate; the bare add is the library's
    chosen = ops.split(llama_layer(weighted=False), 3, T, [HipImplementation(), JitNorms()], Target())
    got = [(c.implementation.library(), c.step.fusion.name) for c in chosen]
    assert got == [("none", "RMS norm"), ("hip", QKV.name), ("hip", PROJECTION.name), ("hip", RESIDUAL.name),
                   ("none", "RMS norm"), ("hip", GATE_UP_SWIGLU.name), ("hip", DOWN_ADD.name)]
    chosen = ops.split(llama_layer(), 3, T, [HipImplementation(), JitNorms()], Target())
    qkv = chosen[1].step
    assert qkv.outputWidth() == DIM + 2 * KV and qkv.weights() == DIM * (DIM + 2 * KV)
    assert [m.weight for m in qkv.matMuls()] == [TensorRole.ATTENTION_QUERY, TensorRole.ATTENTION_KEY,
                                                 TensorRole.ATTENTION_VALUE]


def test_what_the_library_cannot_run_falls_to_the_next_candidate_or_is_named():
    odd = llama_layer(dim=2080)                      # row length not a multiple of 64
    chosen = ops.split(odd, 0, T, [HipImplementation(), JitNorms()], Target())
    assert all(c.implementation.library() == "none" for c in chosen if c.step.matMuls()
               and c.step.matMuls()[0].columns == 2080)
    with pytest.raises(RuntimeError, match=r"no implementation runs RMS_NORM in layer 7 \(ffn\)"):
        ops.split(llama_layer(weighted=False), 7, T, [HipImplementation()], Target(), region="ffn")
    # a per-head norm (Qwen3's query / key norms) is not the row norm the library runs
    per_head = [RmsNorm("q", "q", TensorRole.ATTENTION_NORM, 1e-6, 128, groups=16)]
    with pytest.raises(RuntimeError, match="no implementation runs RMS_NORM"):
        ops.split(per_head, 0, T, [HipImplementation()], Target())
    # an add in front of a norm of some other array is two steps, not the fused one
    apart = [ResidualAdd("y", "xb2"), RmsNorm("x", "xb", TensorRole.FFN_NORM, 1e-5, DIM)]
    assert [c.step.fusion.name for c in ops.split(apart, 0, T, [HipImplementation()], Target())] == [RESIDUAL.name, NORM.name]
    # native libraries switched off (--no-native-libraries), or no matrix cores: never claimed
    for target in (Target(nativeLibraries=False), Target(capabilities=frozenset())):
        chosen = ops.split(llama_layer(), 0, T, [HipImplementation(), JitNorms()], target)
        assert all(c.implementation.library() == "none" for c in chosen)
    # q, k, v reading different inputs are three projections, not one q|k|v
    R = TensorRole
    three = [MatMul(R.ATTENTION_QUERY, "a", "q", 256, 256, T, GGMLType.Q4_K),
             MatMul(R.ATTENTION_KEY, "b", "k", 256, 256, T, GGMLType.Q4_K),
             MatMul(R.ATTENTION_VALUE, "b", "v", 256, 256, T, GGMLType.Q4_K)]
    assert [c.step.fusion.name for c in ops.split(three, 0, T, [HipImplementation()], Target())] == [PROJECTION.name] * 3
    # mixed representations in one fused step are one call (each weight decoded by its own type,
    # DequantizingMatMul.java:53-63); weights of different row lengths are not
    mixed = [MatMul(R.FFN_GATE, "xb", "hb", 512, 256, T, GGMLType.Q4_K),
             MatMul(R.FFN_UP, "xb", "hb2", 512, 256, T, GGMLType.Q6_K), SwiGLU("hb", "hb2", "hb")]
    assert [c.step.fusion.name for c in ops.split(mixed, 0, T, [HipImplementation()], Target())] == [GATE_UP_SWIGLU.name]
    uneven = [MatMul(R.FFN_GATE, "xb", "hb", 512, 256, T, GGMLType.Q4_K),
              MatMul(R.FFN_UP, "xb", "hb2", 512, 512, T, GGMLType.Q4_K), SwiGLU("hb", "hb2", "hb")]
    with pytest.raises(RuntimeError, match="no implementation runs SWIGLU"):
        ops.split(uneven, 0, T, [HipImplementation()], Target())


def test_needs_is_the_workspace_query_and_counts_residency():
    lib = L.load()
    steps = [c.step for c in ops.split(llama_layer(), 0, T, [HipImplementation(), JitNorms()], Target())
             if c.implementation.library() == "hip"]
    need = HipImplementation().needs(steps, Target())
    assert need.residentBytes == 0
    assert need.bytes == lib.jl_gemm_workspace_bytes(T, FFN, 2 * FFN, L.JL_MATH_DEFAULT)
    kept = HipImplementation(residency=True).needs(steps, Target())
    assert kept.bytes == need.bytes
    weights = sum(s.weights() for s in steps)
    assert 2 * weights <= kept.residentBytes <= 2 * weights + 4 * 512 * FFN * 2      # 2 bytes per weight + padding
    assert HipImplementation().needs([], Target()) == ops.BatchPrefillWorkspace.withoutResidencyChoice(0)


def test_records_refuse_what_the_reference_refuses():
    with pytest.raises(ValueError, match="rows and columns must be positive"):
        MatMul(TensorRole.FFN_DOWN, "a", "b", 0, 256, 1, GGMLType.Q8_0)
    with pytest.raises(ValueError, match="batchSize must be positive"):
        MatMul(TensorRole.FFN_DOWN, "a", "b", 256, 256, 0, GGMLType.Q8_0)
    with pytest.raises(ValueError, match="at least one operation"):
        ops.Fusion.of("nothing")
    step = Step(0, T, PROJECTION, (MatMul(TensorRole.FFN_DOWN, "a", "b", 256, 256, T, GGMLType.Q8_0),))
    with pytest.raises(ValueError, match="projection has no SwiGLU"):
        step.first(SwiGLU)
