"""The comparison switches of the library (environment variables read once per process) select kernels that the default
dispatch only takes for other dtypes or shapes.  Each group of switches is set for a child process that runs the
parity tests of the operators concerned: the alternative kernels must meet the same bars on the 16-bit cases too."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

GROUPS = [
    # vector-ALU head mixing for 16 and 32 heads; the general softmax and fused kernels for 16-bit data
    ({"MTA_HEADMIX_NO_MFMA": "1", "MTA_SOFTMAX_NO_PACKED": "1", "MTA_FUSED_FORCE_GENERAL": "1"},
     ["tests/test_gpu_ops.py", "tests/test_gpu_attention.py"],
     "test_headmix_parity or (test_mix_softmax_mix_parity and not f32 and not (case12 or case13 or case14 or case15 or case16 or case17 or case18)) or test_conv_attention_parity "
     "or test_mta_general"),   # (the cases of groups of 16 heads run the same kernel under these switches: left out)
    # another cut of the scores kernel's work items (long / short items of 20 / 7 key blocks, 30 % of a key range short)
    ({"MTA_QK_CHUNK_LONG": "20", "MTA_QK_CHUNK_SHORT": "7", "MTA_QK_SHORT_PERCENT": "30"},
     ["tests/test_gpu_attention.py"], "test_qk_conv_parity or test_mta_headline_route_long_sequence"),
    # fp32-FMA conv kernels (forward, input gradient, weight gradient) for 16-bit data
    ({"MTA_CONV_FORCE_VALU": "1"},
     ["tests/test_gpu_ops.py", "tests/test_gpu_backward.py"],
     "test_conv_parity or test_conv_identity_tap or test_conv_backward_parity"),
    # dense groups of 16 heads in the one-pass conv + mixing entry point on the vector-ALU kernel
    ({"MTA_CONV_MIX16_OFF": "1"}, ["tests/test_gpu_ops.py"], "test_conv_headmix_parity"),
    # P V of small grids on the one-group kernel that large grids run (by default they split the key blocks between two
    # groups of wavefronts)
    ({"MTA_PV_SPLIT": "1"}, ["tests/test_gpu_attention.py"], "test_causal_pv"),
    # mix -> softmax -> mix for groups of 16 heads with a workgroup per row (by default workgroups take lists of rows)
    # the inference route with its score tensors as (B,H,S,S) planes (by default: the triangular layout)
    ({"MTA_SCORE_LAYOUT": "planes"}, ["tests/test_gpu_attention.py"],
     "test_mta_headline or test_mta_use_mask_band or test_mta_use_mask_right_padded or test_mta_use_mask_left_padded "
     "or test_mta_use_mask_key or test_mta_general"),
    # the softmax without weights with a workgroup per row (by default short rows take a wavefront per row)
    ({"MTA_SOFTMAX_NO_WAVE_ROWS": "1"}, ["tests/test_gpu_ops.py"], "test_mix_softmax_mix_parity and not f32 and (case21 or case22 or case23)"),
    ({"MTA_MIX16_NO_ROW_LISTS": "1"}, ["tests/test_gpu_ops.py"], "(test_mix_softmax_mix_parity and not f32 and (case12 or case13 or case14 or case15 or case18)) or test_mix_softmax_mix_dense16"),
    # (the cases with groups of 16 heads, rows of up to 3000 keys: all three kinds of rows)
]


@pytest.mark.parametrize("group", range(len(GROUPS)))
def test_comparison_switches_meet_the_same_bars(group):
    env, files, select = GROUPS[group]
    print(f"switches {sorted(env)}", flush=True)
    cmd = [sys.executable, "-u", "-m", "pytest", *files, "-x", "-q", "-k", select, "-p", "no:cacheprovider",
           "--timeout", "120", "--timeout-method", "thread"]
    r = subprocess.run(cmd, cwd=ROOT, env={**os.environ, **env}, capture_output=True, text=True, timeout=900)
    tail = (r.stdout or "")[-3000:] + (r.stderr or "")[-1000:]
    assert r.returncode == 0, tail
    assert " passed" in r.stdout, tail
