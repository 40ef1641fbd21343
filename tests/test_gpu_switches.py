"""The launch forms that only an environment switch selects (fallback kernels, the older forms kept for comparison) against
the oracle: each case runs a few of the ordinary parity tests in a child process with the switch set -- the library reads
its switches once per process.  One child at a time; a child takes a few seconds."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CASES = [
    ({"LOCAL_HIP_TQ2_KERNEL": "valu", "LOCAL_HIP_X_LIMBS": "3"}, "test_gpu_matvec.py", "baseline_configs or soa"),
    ({"LOCAL_HIP_Q4_IMAGE": "0", "LOCAL_HIP_TQ2_WIDE": "0"}, "test_gpu_matvec.py", "evenly_spaced or long_rows"),
    ({"LOCAL_HIP_TQ2_WIDE_SPLIT": "0"}, "test_gpu_matvec.py", "long_rows"),
    ({"LOCAL_HIP_TQ2_FORCE_SPLIT": "1", "LOCAL_HIP_TQ2_SPLIT6": "0"}, "test_gpu_matvec.py", "reference_payloads and tq2_0"),
    ({"LOCAL_HIP_PREFILL_PW": "4"}, "test_gpu_matmul.py", "prefill_config or large_tiles or weight_tiles"),
    ({"LOCAL_HIP_PREFILL_BF16_PASS": "1"}, "test_gpu_matmul.py", "prefill_config or large_tiles"),
    ({"LOCAL_HIP_MATMUL_SPLITK": "0", "LOCAL_HIP_MATMUL_SKINNY": "0"}, "test_gpu_matmul.py", "decode_batch_matmul or matmul_grouped or tile_boundaries"),
    ({"LOCAL_HIP_ATTN_KERNEL": "valu", "LOCAL_HIP_ATTN_MERGE_ROTATE": "0"}, "test_gpu_attention.py",
     "asymmetric_levels or empty_range or ring_matches or rotated_entry"),
    ({"LOCAL_HIP_ATTN_OCC": "1", "LOCAL_HIP_ATTN_WAVES_PER_SIMD": "3"}, "test_gpu_attention.py", "batched_matches or split_invariance or asymmetric_levels"),
    # hand-overs of two groups forced onto every chunk length (missing and partial groups at both chunk ends), and never used
    ({"LOCAL_HIP_ATTN_PAIR": "1"}, "test_gpu_attention.py", "decode_attention_matches or prefill_matches or batched_matches or "
     "split_invariance or ring_matches or asymmetric_levels or empty_range or attention_sink or randomised_shapes"),
    ({"LOCAL_HIP_ATTN_PAIR": "0"}, "test_gpu_attention.py", "split_invariance or context_sweep_long"),
    ({"LOCAL_HIP_PREFILL_BM": "64", "LOCAL_HIP_SKINNY_MAX_M": "64", "LOCAL_HIP_MATVEC_WG_PER_CU": "1"}, "test_gpu_matmul.py",
     "prefill_config or large_tiles or small_batch_layer_config"),
]


@pytest.mark.parametrize("env,file,expr", CASES, ids=[",".join(f"{k}={v}" for k, v in c[0].items()) for c in CASES])
def test_switched_form_passes_its_parity_tests(env, file, expr):
    child_env = dict(os.environ)
    child_env.update(env)
    cmd = [sys.executable, "-u", "-m", "pytest", os.path.join(ROOT, "tests", file), "-x", "-q", "-m", "gpu", "-k", expr,
           "-p", "no:cacheprovider", "--timeout", "120", "--timeout-method", "thread"]
    print("child:", " ".join(f"{k}={v}" for k, v in env.items()), " ".join(cmd[1:]), flush=True)
    r = subprocess.run(cmd, cwd=ROOT, env=child_env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    tail = "\n".join(r.stdout.splitlines()[-25:])
    assert r.returncode == 0, f"child pytest failed under {env}:\n{tail}"
    assert " passed" in tail and "no tests ran" not in tail, f"nothing ran under {env}:\n{tail}"
