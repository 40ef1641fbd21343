"""The launch forms that only an environment switch selects against the oracle: the fallback kernels (vector-ALU TQ2_0
matvec, vector-ALU attention) that otherwise run only for shapes the matrix-core kernels do not take, the two prefill
attention kernels each on every prefill case (by default the launch size decides between them), and the test aid that
forces the attention kernel's paired hand-overs onto short chunks.  Each case runs a few
of the ordinary parity tests in a child process with the switch set -- the library reads its switches once per
process.  One child at a time; a child takes a few seconds."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CASES = [
    ({"LOCAL_HIP_TQ2_KERNEL": "valu"}, "test_gpu_matvec.py", "baseline_configs or soa or reference_payloads"),
    ({"LOCAL_HIP_ATTN_KERNEL": "valu"}, "test_gpu_attention.py", "asymmetric_levels or empty_range or ring_matches or rotated_entry"),
    ({"LOCAL_HIP_ATTN_PREFILL": "rows"}, "test_gpu_attention.py", "prefill"),
    ({"LOCAL_HIP_ATTN_PREFILL": "tiled"}, "test_gpu_attention.py", "prefill or randomised_shapes"),
    # hand-overs of two groups forced onto every chunk length (missing and partial groups at both chunk ends), and never used
    ({"LOCAL_HIP_ATTN_PAIR": "1"}, "test_gpu_attention.py", "decode_attention_matches or prefill_matches or batched_matches or "
     "split_invariance or ring_matches or asymmetric_levels or empty_range or attention_sink or randomised_shapes"),
    ({"LOCAL_HIP_ATTN_PAIR": "0"}, "test_gpu_attention.py", "split_invariance or context_sweep_long"),
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
