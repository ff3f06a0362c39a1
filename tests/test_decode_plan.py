"""The host runtime's choice of how many splits a step of decoded tokens cuts its keys into
(csrc/host/decode_plan.cpp), on the CPU: the cases it was fitted to, and what it must never do."""
import ctypes
import random

import pytest

from llmengine.engine.scheduler import rounds_order
from llmengine.runtime import native

# the constants of ops.choices.KernelChoices, heads of 64, 8 tiles a request, 256 compute units; a cut costs
# the join and the rotation kernel
ARGS = dict(tiles=8, units=256, head_dim=64, first=1, most=8, tbs=6.0, key_ns=9.5, lone_ns=8.3, piece_us=0.5, apart_us=9.4,
            each_us=1.0, gain=0.05)


def cut(lens, plan_len=0, **kw):
    a = dict(ARGS, **kw)
    lib = native.library()
    return lib.llme_decode_cut((ctypes.c_int * len(lens))(*lens), len(lens), a["tiles"], a["units"], a["head_dim"],
                               max(plan_len, max(lens)), a["first"], a["most"], a["tbs"], a["key_ns"], a["lone_ns"], a["piece_us"],
                               a["apart_us"], a["each_us"], a["gain"])


def test_requests_of_one_length():
    # (measured at the 1B sizes: the best number of splits, or one within 2 % of it)
    assert all(cut([2048] * S) == 1 for S in (17, 24, 32, 33, 40, 48, 64, 65, 96))
    assert [cut([8192] * S) for S in (28, 32, 56, 64, 96, 128)] == [1] * 6
    assert cut([8192] * 17) in (3, 5, 7) and cut([8192] * 20) == 3
    assert cut([8192] * 33) in (4, 6, 7, 8) and cut([8192] * 40) in (3, 4) and cut([8192] * 48) == 2
    assert cut([8192] * 72) in (2, 3, 4)
    assert cut([16384] * 17) >= 3 and cut([16384] * 33) >= 4
    # a cut that costs nothing but its splits is taken earlier; one that may not be taken is not
    assert cut([4096] * 20, apart_us=0.0) > 1 and cut([4096] * 20) == 1
    assert cut([16384] * 33, most=1) == 1


def test_requests_of_different_lengths():
    for lo, hi in ((256, 6144), (1024, 16384)):
        for S in (17, 20, 24):
            rnd = random.Random(S)
            lens = sorted((rnd.randint(lo, hi) for _ in range(S)), reverse=True)
            assert cut(lens) > 1                        # fewer workgroups than units: the long requests are cut
        for S in (33, 36, 40, 48, 65, 72, 96):
            rnd = random.Random(S)
            lens = sorted((rnd.randint(lo, hi) for _ in range(S)), reverse=True)
            lens = [lens[r] for r in rounds_order(S, 32)]
            assert cut(lens) == 1                       # long and short share a unit already
    # one long request among short ones, fewer workgroups than units: it is what the step waits for
    assert cut([16000] + [300] * 19) > 1


def test_few_requests_whose_splits_fill_the_units_once():
    """12 requests, 96 workgroups a split: two splits fill the units once (first=2). Requests of one length keep
    them; with different lengths the short requests' last pieces are empty and a third split is better."""
    free = dict(first=2, most=4, apart_us=0.0)
    assert cut([8192] * 12, **free) == 2 and cut([2048] * 12, **free) == 2
    rnd = random.Random(12)
    lens = sorted((rnd.randint(1024, 16384) for _ in range(12)), reverse=True)
    assert cut(lens, **free) == 3
    assert cut([8192] * 8, first=4, most=6, apart_us=0.0) == 4
    assert cut([300] * 12, first=2, most=4, apart_us=0.0) == 2     # nothing to cut into


def test_limits_and_refusals():
    assert cut([300] * 40) == 1                          # nothing to cut into
    assert cut([100000] * 200) == 1                      # more than ten workgroups a unit
    assert 1 <= cut([100000] * 17) <= 8
    lib = native.library()
    one = (ctypes.c_int * 1)(5)
    assert lib.llme_decode_cut(one, 0, 8, 256, 64, 5, 1, 8, 6.0, 9.5, 8.3, 0.5, 9.4, 1.0, 0.05) == native.BAD_ARGUMENT
    assert lib.llme_decode_cut(one, 1, 0, 256, 64, 5, 1, 8, 6.0, 9.5, 8.3, 0.5, 9.4, 1.0, 0.05) == native.BAD_ARGUMENT
    assert lib.llme_decode_cut(one, 1, 8, 256, 64, 5, 1, 8, 0.0, 9.5, 8.3, 0.5, 9.4, 1.0, 0.05) == native.BAD_ARGUMENT
    assert lib.llme_decode_cut(None, 1, 8, 256, 64, 5, 1, 8, 6.0, 9.5, 8.3, 0.5, 9.4, 1.0, 0.05) == native.BAD_ARGUMENT
    bad = (ctypes.c_int * 2)(5, -1)
    assert lib.llme_decode_cut(bad, 2, 8, 256, 64, 5, 1, 8, 6.0, 9.5, 8.3, 0.5, 9.4, 1.0, 0.05) == native.BAD_ARGUMENT
