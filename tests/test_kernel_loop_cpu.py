"""The scoring kernel's own op loop (superscaler_amd/csrc/ace_score_loop.h: group loads, padding,
row windows, deferred stage tails, single-stage ranges) and the plan-editing kernels
(csrc/ace_edit_kernels.h: move descriptors, check_recompute's selection) compiled for the CPU and run with every
array flush against an inaccessible page, one child process per case: an index past an array ends
the child with SIGSEGV here, where it costs nothing, instead of as a memory fault on a GPU.
Results are compared with the state-machine emulation (which the other CPU tests pin to the oracle)."""
import os
import subprocess
import sys

import pytest

from superscaler_amd import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CASES = [(name, mode, 96 if name != "gpt3_175b" else 24) for name in synth.WORKLOADS
         for mode in ("plain", "breakdown", "ranged", "junk", "moves", "recompute")] + [("-", "golden_resnet", 0),
                                                                                       ("gpt3_1_3b", "collective", 96),
                                                                                       ("wresnet_1b", "collective", 96)]


@pytest.mark.parametrize("workload,mode,n", CASES, ids=[f"{c[0]}-{c[1]}" for c in CASES])
def test_kernel_loop_stays_inside_its_arrays(workload, mode, n):
    from tests.helpers import emu_lib
    emu_lib()                                   # build once, in this process
    proc = subprocess.run([sys.executable, "-m", "tests.emu.guarded_case", workload, mode, str(n)], cwd=ROOT,
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert proc.returncode == 0 and proc.stdout.strip().endswith("ok"), \
        f"child ended with {proc.returncode} (negative: killed by that signal)\n{proc.stdout[-2000:]}"
