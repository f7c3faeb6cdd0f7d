"""reef_ops_conv2d_noalloc: the convolution entry point that allocates nothing (its split-K
partial tiles and arrival counters live in a fixed device array of the library) must give
exactly the bits of reef_ops_conv2d, call after call, although every call reuses the array."""
import numpy as np
import pytest

from reef_amd import binding as B
from tests.helpers import max_rel_err, REL_TOL
from tests.test_gpu_conv_op import run_case, RNG

pytestmark = pytest.mark.gpu


def both(case):
    state = RNG.bit_generator.state
    st_a, got_a, ref = run_case(case, noalloc=False)
    RNG.bit_generator.state = state          # the same random operands for the second entry point
    st_n, got_n, _ = run_case(case, noalloc=True)
    assert st_a == 0 and st_n == 0, B.last_error()
    np.testing.assert_array_equal(got_n, got_a)
    assert max_rel_err(got_n, ref) <= REL_TOL


def test_no_alloc_equals_allocating_entry_point_twice_in_a_row():
    B.ops_init()
    # both layers split K (partial tiles and counters in the scratch array); the second is smaller,
    # so it finds the first call's leftovers in the array
    both((512, 14, 14, 256, 3, 1, 1, 1, True, True))
    both((256, 7, 7, 64, 3, 1, 1, 1, True, False))
    both((1024, 14, 14, 256, 1, 1, 0, 1, True, False))
    both((128, 7, 7, 32, 1, 1, 0, 0, False, False))
    # a layer without a split needs no scratch at all
    both((64, 56, 56, 64, 3, 1, 1, 1, True, False))


def test_no_alloc_needs_init_and_states_its_limit():
    L = B.lib()
    L.reef_ops_scratch_bytes.restype = __import__("ctypes").c_size_t
    assert L.reef_ops_scratch_bytes() == 4 << 20
    # A call in a process where reef_ops_init has not run is refused before anything is launched
    # (set-up -- loading the kernels, finding this GPU's copy of the array -- is never done by
    # the entry point that must not allocate).  In a process of its own: this one has run init.
    import subprocess
    import sys
    code = (
        "import ctypes, sys\n"
        "from reef_amd import binding as B\n"
        "d = B.Conv2dDesc(256, 14, 14, 256, 3, 3, 1, 1, 1, 1, 1)\n"
        "p = ctypes.c_void_p(4096)\n"      # never dereferenced: the refusal comes first
        "st = B.lib().reef_ops_conv2d_noalloc(ctypes.byref(d), p, p, None, None, p, None)\n"
        "print(st, B.last_error())\n"
        "sys.exit(0 if st == 1 and 'reef_ops_init has not run' in B.last_error() else 3)\n")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300,
                       cwd=__import__("os").path.dirname(__import__("os").path.dirname(__import__("os").path.abspath(__file__))))
    assert r.returncode == 0, (r.stdout, r.stderr)
    # The size check of the entry point is a guard that no shape reaches today: its plan puts at most
    # 256 workgroups on a split layer and a workgroup's tile has at most 64 x 64 outputs, so the
    # partial tiles never exceed 256 x 4096 floats = the 4 MiB array, and a split layer has at most
    # 128 tiles against 16384 counters.  The largest such layer goes through and matches:
    B.ops_init()
    both((2048, 7, 7, 2048, 1, 1, 0, 0, False, False))
