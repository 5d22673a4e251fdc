"""The arrival protocol of the GEMM's K split (comfyui-int8-fast_amd/csrc/splitk_protocol.h), compiled for the
host and driven through every interleaving that matters: it is plain C shared by the kernel and this test."""
import ctypes
import itertools
import os
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "comfyui-int8-fast_amd", "csrc", "splitk_protocol.h")

SHIM = """
#include "%s"
uint32_t t_arrive(uint32_t word, uint32_t tag, uint32_t splits, uint32_t *before) { return splitk_arrive(word, tag, splits, before); }
uint32_t t_tag(uint32_t n) { return splitk_tag(n); }
"""


@pytest.fixture(scope="module")
def proto():
    d = tempfile.mkdtemp(prefix="i8f_splitk_")
    src, so = os.path.join(d, "shim.c"), os.path.join(d, "shim.so")
    with open(src, "w") as f:
        f.write(SHIM % HEADER)
    subprocess.run(["gcc", "-O1", "-shared", "-fPIC", "-o", so, src], check=True)
    lib = ctypes.CDLL(so)
    lib.t_arrive.restype = ctypes.c_uint32
    lib.t_arrive.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32)]
    lib.t_tag.restype = ctypes.c_uint32
    lib.t_tag.argtypes = [ctypes.c_uint32]

    def arrive(word, tag, splits):
        before = ctypes.c_uint32()
        return lib.t_arrive(word, tag, splits, ctypes.byref(before)), before.value
    return arrive, lib.t_tag


def run_launch(arrive, word, tag, splits):
    """All slices of one launch arrive one after the other (a compare-and-swap serialises them): -> (final word,
    how many slices saw themselves as the last one)."""
    lasts = 0
    for _ in range(splits):
        word, before = arrive(word, tag, splits)
        assert 0 <= before < splits
        lasts += before + 1 == splits
    return word, lasts


def test_clean_word_has_exactly_one_last_slice(proto):
    arrive, _ = proto
    for splits in range(2, 9):
        word, lasts = run_launch(arrive, 0, 7, splits)
        assert lasts == 1 and word == (7 << 8) | splits


@pytest.mark.parametrize("splits", [2, 3, 5, 8])
def test_leftover_words_do_not_poison_the_next_launch(proto, splits):
    """Whatever an earlier launch left behind (another tag with any count, a count this launch's slices cannot
    leave, garbage), the next launch has exactly one last slice."""
    arrive, _ = proto
    tag = 0x00beef
    leftovers = [(other << 8) | c for other in (1, 0x00bee0, 0xffffff) for c in range(0, 256, 1 if splits < 4 else 17)]
    leftovers += [c for c in range(256)] + [(tag << 8) | c for c in (0, splits, splits + 1, 255)] + [0xffffffff, 0x80000000]
    for word in leftovers:
        final, lasts = run_launch(arrive, word, tag, splits)
        assert lasts == 1, hex(word)
        assert final == (tag << 8) | splits


def test_replay_with_the_same_tag_after_the_reset_and_after_a_lost_reset(proto):
    """A captured launch is replayed with its tag: after the last slice's reset (word 0) and also if that reset was
    lost (word = tag, splits) the replay counts from one again."""
    arrive, _ = proto
    for word in (0, (9 << 8) | 4):
        assert run_launch(arrive, word, 9, 4) == ((9 << 8) | 4, 1)


def test_interleaved_arrivals_of_two_tiles_are_independent_and_any_order_gives_one_last(proto):
    arrive, _ = proto
    for order in itertools.permutations(range(4)):
        word, lasts = 0x5a5a5a5a, []
        for _slice in order:
            word, before = arrive(word, 3, 4)
            lasts.append(before)
        assert sorted(lasts) == [0, 1, 2, 3]


def test_tags_are_nonzero_24_bit_and_distinct_for_consecutive_launches(proto):
    _, tag = proto
    seen = [tag(n) for n in list(range(1000)) + [0xfffffe, 0xffffff, 0x1000000, 0xffffffff]]
    assert all(0 < t <= 0xffffff for t in seen)
    assert len(set(seen[:1000])) == 1000
    assert tag(0xfffffe) != tag(0xffffff)
