"""CPU: the jump-ahead polynomials of brainstorm_amd/csrc/mt_jump.h against NumPy's generator.

The library cuts a long mask draw into segments and forms each segment's 624-word start block as an
XOR combination of the stream (w[d + j] = XOR of w[i + j] over the set coefficients of x^d mod
x*phi(x)). The check program forms blocks exactly that way from a key taken from
numpy.random.RandomState; the expected blocks are the keys RandomState itself holds after drawing
that far. Nothing here needs a GPU."""
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("mt_jump") / "mt_jump_check")
    subprocess.run(["g++", "-O2", "-std=c++17", "-o", exe, os.path.join(HERE, "mt_jump_check.cpp")], check=True)
    return exe


def key_after_blocks(seed, start_doubles, blocks):
    """Key of RandomState(seed) `blocks` 624-word blocks after the block it holds once start_doubles are drawn."""
    rs = np.random.RandomState(seed)
    if start_doubles:
        rs.random_sample(start_doubles)
    key0, pos0 = rs.get_state()[1].copy(), rs.get_state()[2]
    # draw up to two words into the block that lies `blocks` further on
    rs.random_sample((624 * blocks - pos0) // 2 + 1)
    state = rs.get_state()
    assert 0 < state[2] <= 3
    return key0, state[1]


@pytest.mark.parametrize("seed,start,blocks_per_segment,count", [(0, 0, 16, 3), (123, 1000, 1, 2), (7, 5, 211, 2),
                                                                  (4294967295, 311, 32, 4)])
def test_jumped_blocks_are_numpys(checker, seed, start, blocks_per_segment, count):
    key0, _ = key_after_blocks(seed, start, 1)
    out = subprocess.run([checker, str(624 * blocks_per_segment), str(count)], input="\n".join(str(int(v)) for v in key0),
                         capture_output=True, text=True, check=True).stdout.split()
    got = np.array(out, dtype=np.uint64).astype(np.uint32).reshape(count, 624)
    for k in range(1, count + 1):
        _, want = key_after_blocks(seed, start, blocks_per_segment * k)
        np.testing.assert_array_equal(got[k - 1], want, err_msg="block %d segments ahead" % k)
