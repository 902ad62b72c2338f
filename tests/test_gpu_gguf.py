"""GPU: weights uploaded straight from a mapped GGUF file decode and multiply like the same blocks
uploaded from memory."""
import numpy as np
import pytest

import gguf_writer as W
from gpu_util import bits_equal, magnitude, rel_err, say
from oracle import pyoracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from jitllm_amd.runtime import Context
    c = Context(0)
    yield c
    c.close()


def test_upload_from_file_then_project(ctx, tmp_path):
    from jitllm_amd import synthetic
    from jitllm_amd.gguf import GGUF
    from jitllm_amd.projections import QuantizedProjections, TornadoWorkspace
    say("gguf upload")
    d, n = 96, 2048
    raws = {"blk.0.attn_q.weight": (O.Q8_0, synthetic.weight(O.Q8_0, d, n, seed=901)),
            "blk.0.ffn_up.weight": (O.Q4_0, synthetic.weight(O.Q4_0, d, n, seed=902)),
            "blk.0.ffn_down.weight": (O.Q4_K, synthetic.weight(O.Q4_K, d, n, seed=903)),
            "output.weight": (O.Q6_K, synthetic.weight(O.Q6_K, d, n, seed=906)),
            "blk.0.attn_v.weight": (O.Q5_K, synthetic.weight(O.Q5_K, d, n, seed=907)),
            "blk.1.ffn_down.weight": (O.Q4_1, synthetic.weight(O.Q4_1, d, n, seed=908)),
            "blk.1.attn_k.weight": (O.Q5_0, synthetic.weight(O.Q5_0, d, n, seed=909)),
            "blk.1.attn_q.weight": (O.IQ4_XS, synthetic.weight(O.IQ4_XS, d, n, seed=910))}
    tensors = [("pad.me", (5,), 24, np.arange(5, dtype=np.uint8))]       # pushes the next offset off 32
    tensors += [(name, (n, d), int(t), raw) for name, (t, raw) in raws.items()]
    path = tmp_path / "m.gguf"
    W.write_gguf(path, [("general.architecture", W.STRING, "llama")], tensors, alignment=64)
    x = synthetic.activations(n, seed=904)
    with GGUF(path) as g:
        for name, (t, raw) in raws.items():
            w = g.load_weight(ctx, name)
            assert (w.rows, w.cols, int(w.data_type())) == (d, n, int(t))
            assert bits_equal(w.dequantize(), O.dequant(t, raw))
            out = ctx.float_array(d, fill=-1.0)
            QuantizedProjections(ctx, TornadoWorkspace()).floatMatvec(ctx.from_numpy(x), out, w, n, d)
            ctx.sync()
            assert rel_err(out.get(), O.matmul(t, raw, x, d, n), magnitude(t, raw, x, d, n)) < 2e-5


def test_upload_refuses_other_types_and_truncated_files(ctx, tmp_path):
    from jitllm_amd._lib import JitllmHipError, UnsupportedProjection
    from jitllm_amd import synthetic
    from jitllm_amd.gguf import GGUF
    say("gguf refusals")
    d, n = 8, 256
    raw = synthetic.weight(O.Q8_0, d, n, seed=905)
    path = tmp_path / "m.gguf"
    W.write_gguf(path, [], [("norm.weight", (n,), 0, np.ones(n, dtype=np.float32)),
                            ("emb.weight", (n, 3), 9, np.zeros(3 * 8 * 40, dtype=np.uint8)),   # Q8_1
                            ("q.weight", (n, d), 8, raw)], truncate_data_by=100)
    with GGUF(path) as g:
        with pytest.raises(UnsupportedProjection, match="ggml type 0"):
            g.load_weight(ctx, "norm.weight")
        with pytest.raises(UnsupportedProjection, match="ggml type 9"):
            g.load_weight(ctx, "emb.weight")
        with pytest.raises(JitllmHipError, match="runs past the end of the file"):
            g.load_weight(ctx, "q.weight")
        with pytest.raises(JitllmHipError, match="no tensor absent"):
            g.load_weight(ctx, "absent")
