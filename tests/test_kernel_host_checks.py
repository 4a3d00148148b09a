"""What the kernel library decides on the host, checked without a GPU (the library's host functions run
anywhere): the search that the workgroups of an `uneven` decoding attention launch make for their split length
always ends within its budget of tries, for any lengths within the launch's bound."""
import ctypes
import random

import pytest

from longbow_quarrel_amd import build


@pytest.fixture(scope="module")
def lib():
    return ctypes.CDLL(build.ensure_built())


def tries(lib, positions, nkv, max_len):
    arr = (ctypes.c_int * len(positions))(*positions)
    return lib.lq_attention_unit_search(arr, len(positions), nkv, max_len)


def test_the_units_of_an_uneven_decoding_launch_always_find_their_split_length(lib):
    rnd = random.Random(5)
    worst = 0
    taken = 0
    for rows in list(range(2, 65)):
        for nkv in (1, 2, 3, 8, 16, 64):
            for max_len in (512, 1000, 1024, 1025, 4096, 8192, 40000, 131072, 1 << 20):
                cases = [
                    [max_len - 1] * rows,                                   # every sequence as long as the bound
                    [max_len - 1] + [0] * (rows - 1),                       # one long, the others new
                    [max_len - 1] + [255] * (rows - 1),
                    [max_len - 1, max_len // 2] + [256] * (rows - 2),
                    [rnd.randrange(max_len) for _ in range(rows)],
                    [min(max_len - 1, 256 * rnd.randrange(1, 8) - 1) for _ in range(rows)],  # splits filled to the brim
                ]
                for positions in cases:
                    n = tries(lib, positions, nkv, max_len)
                    assert n >= 0, (rows, nkv, max_len, positions[:4])
                    worst = max(worst, n)
                    taken += n > 0
    assert taken > 1000  # the sweep did meet launches that take the units' way
    assert worst <= 1024


def test_launches_that_do_not_share_out_by_units_say_so(lib):
    assert tries(lib, [5000], 8, 8192) == 0            # one sequence
    assert tries(lib, [100] * 65, 8, 8192) == 0        # more sequences than a wave has lanes
    assert tries(lib, [100, 50], 8, 0) == 0            # no bound
