"""Run tests of the GPU suite on the lane-level CPU emulation instead of a device:

    python tests/emu/run_on_emulator.py [pytest arguments]

The package's ctypes loader is pointed at tests/emu/libnervana_emu.so (the kernel sources compiled
for the host, see shim/hip/hip_runtime.h) for this process only; the emulation reports one device,
so the tests marked `gpu` run.  Generated elementwise kernels are compiled with the host compiler
against the same stand-in headers.  Test infrastructure: slow, and it says nothing about speed."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, HERE)

import emu  # noqa: E402

emu.build()

from nervanagpu_amd import _lib  # noqa: E402

_lib.LIB_PATH = emu.LIB
lib = _lib.load()
lib.emu_set_cus(int(os.environ.get("EMU_CUS", "8")))
lib.emu_set_late_loads(int(os.environ.get("EMU_LATE_LOADS", "1")))
lib.emu_set_shuffle(int(os.environ.get("EMU_SHUFFLE", "5")))

import pytest  # noqa: E402

sys.exit(pytest.main(sys.argv[1:]))
