"""The plain-C harness (flash-attn-rtx5060_amd/host/fa_harness.c, the role of the reference's main()):
run the binary on the GPU, read back what it dumped, and check it against the CPU oracle."""
import json
import os
import subprocess

import numpy as np
import pytest

from parity_util import assert_within, errors, make_inputs, sample_rows

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("args,shape,dtype,causal,wl,seed", [
    (["--config", "c1"], (1, 4, 256, 64), 0, False, -1, 27),
    (["--B", "2", "--N", "3", "--S", "1024", "--d", "128", "--bf16", "--causal", "--window-left", "200", "--seed", "5"],
     (2, 3, 1024, 128), 1, True, 200, 5),
    (["--B", "1", "--N", "8", "--S", "1024", "--d", "64", "--causal", "--alibi", "--seed", "6"],
     (1, 8, 1024, 64), 0, True, -1, 6),
    (["--B", "1", "--N", "4", "--S", "640", "--d", "128", "--causal", "--dropout", "0.1", "--seed", "8"],
     (1, 4, 640, 128), 0, True, -1, 8),
])
def test_harness_output_matches_oracle(fa, oracle, tmp_path, args, shape, dtype, causal, wl, seed):
    assert os.path.exists(fa.HARNESS_PATH), "fa_harness has not been built"
    prefix = str(tmp_path / "run")
    proc = subprocess.run([fa.HARNESS_PATH, *args, "--iters", "3", "--warmup", "1", "--dump", prefix],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    report = json.loads(proc.stdout.strip().splitlines()[-1])
    B, H, S, D = shape
    assert (report["B"], report["N"], report["S"], report["d"]) == shape and report["nonfinite_outputs"] == 0
    assert report["algorithmic_flops"] == pytest.approx(fa.lib().fa_algorithmic_flops(B, H, S, D, int(causal), wl, -1))
    q, k, v = (np.fromfile(f"{prefix}.{t}.bin", dtype=np.uint16).reshape(shape) for t in "qkv")
    # the harness generates its inputs with the same seeded generator the tests use
    q2, k2, v2 = make_inputs(fa, shape, dtype, seed)
    assert np.array_equal(q, q2) and np.array_equal(k, k2) and np.array_equal(v, v2)
    o = np.fromfile(f"{prefix}.o.bin", dtype=np.uint16).reshape(-1, D)
    lse = np.fromfile(f"{prefix}.lse.bin", dtype=np.float32)
    rows = sample_rows(shape, 1024, seed)
    slopes = None
    if "--alibi" in args:       # the slopes of the reference's main() (src/main.cu:38-42)
        slopes = np.fromfile(f"{prefix}.slopes.bin", dtype=np.float32)
        assert np.array_equal(slopes, (-np.power(2.0, -8.0 / H * (np.arange(H) + 1))).astype(np.float32))
    drop = (fa.lib().fa_dropout_threshold(0.1), 48) if "--dropout" in args else (0, 0)   # seed 48: main.cu:93
    o_ref, lse_ref = oracle.rows(q, k, v, rows, dtype, None, causal, wl, -1, slopes, dropout=drop)
    err = errors(oracle.to_f32(o[rows], dtype), oracle.to_f32(o_ref, dtype), lse[rows], lse_ref)
    assert_within(err, dtype, f"harness {args}")


@pytest.mark.parametrize("args,shape,dtype,causal,wl,seed", [
    (["--config", "c1"], (1, 4, 256, 64), 0, False, -1, 27),
    (["--B", "1", "--N", "3", "--S", "500", "--d", "128", "--causal", "--alibi", "--dropout", "0.1", "--seed", "9"],
     (1, 3, 500, 128), 0, True, -1, 9),
])
def test_harness_backward_matches_gradient_oracle(fa, oracle, tmp_path, args, shape, dtype, causal, wl, seed):
    """--backward: fa_bwd called from plain C on the forward pass's O and logsumexp; the dumped gradients against
    the fp64 gradient oracle (dO comes from the same seeded generator, seed + 1000)."""
    prefix = str(tmp_path / "run")
    proc = subprocess.run([fa.HARNESS_PATH, *args, "--backward", "--iters", "2", "--warmup", "1", "--dump", prefix],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    lines = proc.stdout.strip().splitlines()
    report = json.loads(lines[-1])
    B, H, S, D = shape
    assert report["config"].endswith("backward") and report["nonfinite_gradients"] == 0
    assert report["algorithmic_flops"] == pytest.approx(2.5 * json.loads(lines[-2])["algorithmic_flops"])
    q, k, v, do = (np.fromfile(f"{prefix}.{t}.bin", dtype=np.uint16).reshape(shape) for t in ("q", "k", "v", "do"))
    do2, _, _ = make_inputs(fa, shape, dtype, seed + 1000)
    assert np.array_equal(do, do2)
    slopes = np.fromfile(f"{prefix}.slopes.bin", dtype=np.float32) if "--alibi" in args else None
    drop = (fa.lib().fa_dropout_threshold(0.1), 48) if "--dropout" in args else (0, 0)
    want = oracle.bwd_f64(q, k, v, do, dtype, None, causal, wl, -1, slopes, dropout=drop)
    grow = 256.0 / (256 - drop[0])
    for name, ref in zip(("dq", "dk", "dv"), want):
        got = oracle.to_f32(np.fromfile(f"{prefix}.{name}.bin", dtype=np.uint16).reshape(shape), dtype).astype(np.float64)
        rel = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
        print("harness backward", args[:2], name, rel)
        assert np.isfinite(got).all() and rel <= 1e-3 * grow, (name, rel)
