"""bench.py's accounting, without a GPU: the algorithmic bytes it divides by are the ones the
benchmark is defined on (weight blocks in the file's layout + fp32 input + fp32 output, once each),
and a run on more than one GPU is refused in words."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_algorithmic_bytes_of_the_decode_set():
    import bench
    # one 2048 x 2048 Q8_0 projection: 4 456 448 B of blocks + 8 192 B in + 8 192 B out
    assert bench.q8_bytes(2048, 2048) == 4_456_448
    assert bench.gemv_bytes(2048, 2048) == 4_472_832
    # the vocabulary projection, a layer's seven projections, a whole token
    assert bench.gemv_bytes(bench.VOCAB, bench.DIM) == 279_606_272
    per_layer = (2 * bench.gemv_bytes(bench.DIM, bench.DIM) + 2 * bench.gemv_bytes(bench.KV_DIM, bench.DIM)
                 + 2 * bench.gemv_bytes(bench.HIDDEN, bench.DIM) + bench.gemv_bytes(bench.DIM, bench.HIDDEN))
    assert per_layer == 64_794_624
    assert bench.decode_bytes() == 16 * 64_794_624 + 279_606_272 == 1_316_320_256
    # the launch the roofline block is about: gate and up, each counted as a projection of its own
    assert 2 * bench.gemv_bytes(bench.HIDDEN, bench.DIM) == 35_733_504
    # the other block layouts: Q4_0 18 bytes per 32 weights, Q4_K 144 per 256
    assert bench.gemv_bytes(4096, 4096, 18, 32) == 4096 * 128 * 18 + 2 * 4 * 4096 == 9_469_952
    assert bench.gemv_bytes(14336, 4096, 18, 32) == 33_103_872
    assert bench.gemv_bytes(1024, 4096, 18, 32) == 2_379_776


def test_more_than_one_gpu_is_refused_in_words():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in (proc.stdout + proc.stderr)
    assert not proc.stdout.strip().startswith("{")
