"""No lane of a matrix-product kernel fetches outside its operand (CPU).

A fetch whose result is discarded (a row beyond the matrix, k beyond a wave's range) changes no
value, so no comparison of results can see where it went; it faults only when the tensor ends
where its mapping ends.  The kernels take their address arithmetic from ``csrc/addressing.h``;
``tests/cpp/load_bounds.cpp`` includes the same header, walks every block, wave, lane and step of
the weight-streaming kernels (row-major and tiled weights) and of the two tile kernels (their
buffer descriptors and lane offsets) for a sweep of shapes, and the key and value fetches of the
attention kernels' chunks (pages that are there, missing, or no pages of the pool) for every head
size, and checks every fetch.
"""
import os
import subprocess

import pytest

from photon_infer_amd.ops import build, fast

HERE = os.path.dirname(os.path.abspath(__file__))

# shapes that once sent a discarded fetch past the last row (k-ranges shorter than one step of 64
# in some wave: the hidden and intermediate sizes of tiny models), and the kernel tests' own shapes
SHORT_RANGES = [(4, 50, 160), (9, 40, 344), (12, 776, 272), (3, 64, 200), (16, 33, 8), (1, 128, 96)]
KERNEL_TEST_SHAPES = [(1, 14, 3), (2, 2, 3), (5, 176, 64), (33, 100, 72), (64, 384, 128), (70, 1001, 96), (1, 256, 64),
                      (130, 64, 200), (257, 320, 136), (8, 2048, 512), (300, 520, 264), (40, 200, 1032), (64, 72, 520),
                      (48, 1001, 96), (35, 130, 2048)]
MODEL_SHAPES = [(m, n, k) for m in (1, 8, 16, 33, 64, 128, 2048) for n, k in ((3072, 2048), (2048, 2048), (16384, 2048), (2048, 8192))]


@pytest.fixture(scope="module")
def program(tmp_path_factory):
    out = tmp_path_factory.mktemp("bounds") / "load_bounds"
    return build.build_host_program([os.path.join(HERE, "cpp", "load_bounds.cpp")], str(out), extra_flags=["-O2"])


def _args(shapes):
    """Each shape with the split counts that the dispatch rules give it, and a few more."""
    out = []
    for m, n, k in shapes:
        if k % 8:
            continue                      # such a product goes to the general kernel
        wanted = {1, 2, 3, fast._skinny_splits(m, n, k) if m <= fast.SKINNY_MAX_ROWS else fast._tile_splits(m, n, k)}
        for s in sorted(wanted):
            if s == 1 or k // s >= 8:
                out += [m, n, k, s]
    return [str(v) for v in out]


def test_every_fetch_of_the_product_kernels_lies_inside_its_operand(program):
    r = subprocess.run([program] + _args(SHORT_RANGES + KERNEL_TEST_SHAPES + MODEL_SHAPES), capture_output=True, text=True, timeout=600)
    assert r.returncode == 0 and r.stdout.startswith("ok "), r.stdout + r.stderr
    assert int(r.stdout.split()[1]) > 10**9          # the sweep did walk the kernels


@pytest.mark.parametrize("shape", SHORT_RANGES[:4])
def test_the_check_sees_the_stand_in_address_that_once_left_the_row(program, shape):
    """The negative control: with the stand-in of a lane beyond a partial step put back to what
    it was (the range's start plus the lane's own offset), the same walk reports a fetch outside
    its row for each of the shapes that the mistake concerned, and passes them as they are now."""
    args = _args([shape])
    good = subprocess.run([program, "only"] + args, capture_output=True, text=True, timeout=120)
    assert good.returncode == 0, good.stdout
    bad = subprocess.run([program, "old-standin", "only"] + args, capture_output=True, text=True, timeout=120)
    assert bad.returncode == 1 and "outside its row" in bad.stdout, bad.stdout
