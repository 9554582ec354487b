"""Every kernel that only runs when another one is switched off (QMM_DISABLE) or when QMM_Q4K_TILE / QMM_Q4K_PLANES /
QMM_Q4_0_PLANES / QMM_Q4K_LANES_ROWS / QMM_Q6K_MM / QMM_Q5K_MM force it: each
setting gets a child process (the library reads its environment once), which checks a fixed set of shapes of all
four encodings against the oracle."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))

SETTINGS = [
    # first-choice kernels off: the second kernel of every dispatch chain
    {"QMM_DISABLE": "q4k_lanes,q4k_lanes_rows,q4k_mm,q4k_tile,q4k_gemm64,q4_0_stream,q4_0_small,q4_0_planes,q6k_lanes,q6k_mm,kquant_planes,gptq_mm"},
    # ... and the second choices too: row kernels, the K-chunk kernel off, slab kernel off
    {"QMM_DISABLE": "q4k_lanes,q4k_lanes_rows,q4k_stream,q4k_mm,q4k_kc,q4k_tile,q4_0_stream,q4_0_small,q4_0_planes,q4_0_wide,q6k_lanes,q6k_mm,q6k_slab,kquant_planes,gptq_mm"},
    # ... down to the first-version kernels of every encoding
    {"QMM_DISABLE": "q4k_lanes,q4k_lanes_rows,q4k_stream,q4k_rows_v2,q4k_mm,q4k_kc,q4k_tile,q4_0_stream,q4_0_planes,q4_0_mfma,q6k_lanes,q6k_mm,q6k_slab,"
                    "q6k_staged,kquant_planes,gptq_mm,gptq_cols"},
    # the tile kernel on shapes it does not get by itself
    {"QMM_Q4K_TILE": "1"},
    # the plane GEMMs of Q4_K and Q4_0, the 2..4-row decode kernel of Q4_K and the small-batch kernels of Q6_K and Q5_K likewise
    {"QMM_Q4K_PLANES": "1", "QMM_Q4_0_PLANES": "1", "QMM_Q4K_LANES_ROWS": "1", "QMM_Q6K_MM": "1", "QMM_Q5K_MM": "1"},
    # the kernels that the 2..4-row decode kernel of Q4_K and the small-batch kernels of Q6_K and Q5_K take small batches from
    {"QMM_DISABLE": "q4k_lanes_rows,q6k_mm,q5k_mm"},
    # large prefill shapes without the plane GEMM on 256 x 256 tiles: Q4_K tile kernel, GPTQ GEMM, Q5_K planes on 256 x 128 tiles
    {"QMM_DISABLE": "planes_wide,planes_quarters"},
    # ... and Q4_K / GPTQ alone kept off the planes
    {"QMM_DISABLE": "q4k_planes,gptq_planes"},
    # the plain calls of Q4_K decode and small batch through the kernels that take several matrices
    {"QMM_DISABLE": "q4k_lanes_plain,q4k_mm_plain"},
    # the small-batch kernels of Q5_K and Q6_K with the rounds of a long K one after the other in each workgroup
    {"QMM_DISABLE": "kquant_mm_rounds_grid"},
    # GPTQ decode on few columns through the kernel with 64 columns per workgroup
    {"QMM_DISABLE": "gptq_cols16"},
]


@pytest.mark.parametrize("setting", SETTINGS, ids=lambda s: ";".join(f"{k}={v}" for k, v in s.items())[:60])
def test_fallback_kernels_match_the_oracle(setting):
    env = dict(os.environ)
    env.update(setting)
    proc = subprocess.run([sys.executable, os.path.join(HERE, "fallback_child.py")], env=env, capture_output=True, text=True,
                          timeout=600)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    assert proc.stdout.count(": ok") == 35, proc.stdout
