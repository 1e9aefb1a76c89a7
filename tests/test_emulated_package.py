"""A slice of the GPU parity suite run on the lane-level CPU emulation (tests/emu): the package's ctypes
loader is pointed at the emulated library in a child process, the emulation reports one device, and the
selected `gpu` tests run unchanged: the Python surface, the C ABI, the compiled kernels and the generated
elementwise kernels (compiled with the host compiler against the stand-in headers), with LDS-bound loads
landing as late as the kernels' wait counts allow and shuffled scheduling.  The selection is what finishes
in about two minutes; `python tests/emu/run_on_emulator.py <pytest arguments>` runs anything else."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SELECTION = [
    ("tests/test_gpu_pool.py", "full_compare or l2 or errors or rectifier"),
    ("tests/test_gpu_aux.py", ""),
    ("tests/test_gpu_ew.py", "math_matrix or unary_ops or argmax_ties or broadcast_transpose or fill_copy or take_and_onehot "
                             "or rand_and_dropout or compensated_sum or (batchnorm_expression and not 8192 and not 20000)"),
]


def _run(path, expr):
    cmd = [sys.executable, os.path.join(ROOT, "tests", "emu", "run_on_emulator.py"), os.path.join(ROOT, path), "-x", "-q",
           "-p", "no:cacheprovider"]
    if expr:
        cmd += ["-k", expr]
    done = subprocess.run(cmd, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=1500)
    tail = done.stdout.decode("utf-8", "replace")[-3000:]
    assert done.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail, tail


def test_pooling_suite_on_the_emulator():
    _run(*SELECTION[0])


def test_data_movement_suite_on_the_emulator():
    _run(*SELECTION[1])


def test_elementwise_suite_on_the_emulator():
    _run(*SELECTION[2])
