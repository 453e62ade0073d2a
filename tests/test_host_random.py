"""The host library's java.util.Random twin (used to build seeded model weights) against the
oracle's independent restatement and the JDK's known outputs; the multi-threaded tensor fill
must be bit-identical to the sequential stream."""
import json
import os

import numpy as np

from deepj_amd import JavaRandom
from oracle import cpu_ref as ref

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))["java_random"]


def test_known_jdk_outputs():
    assert JavaRandom(42).nextInt() == GOLD["next_int_seed42"]
    r = JavaRandom(42)
    assert [r.nextInt(10) for _ in range(5)] == GOLD["next_int_bound10_seed42"]
    assert JavaRandom(0).nextGaussian() == GOLD["next_gaussian_seed0"]
    r = JavaRandom(42)
    assert [r.nextGaussian() for _ in range(4)] == GOLD["next_gaussian_seed42"]
    assert list(JavaRandom(7).ints(8, 256)) == GOLD["prompt_seed7_bound256"]
    assert JavaRandom(5).nextFloat() == ref.JavaRandom(5).next_float()


def test_parallel_fill_is_bit_identical_to_the_sequential_stream():
    n = 300_001                                     # odd: the last pair's second value must stay cached
    for seed in (42, 43, -7):
        a = JavaRandom(seed)
        b = ref.JavaRandom(seed)
        x1 = a.tensor(1, n, threads=7)
        y1 = b.tensor(1, n)
        assert np.array_equal(x1.view(np.int32), y1.view(np.int32))
        # the stream continues correctly after a parallel fill (cached value, LCG position)
        assert a.nextGaussian() == b.next_gaussian()
        x2 = a.tensor(3, 70_000, threads=3)
        y2 = b.tensor(3, 70_000)
        assert np.array_equal(x2.view(np.int32), y2.view(np.int32))
        assert a.nextInt(1000) == b.next_int(1000)


def test_small_fills_and_scale():
    a, b = JavaRandom(1), ref.JavaRandom(1)
    assert np.array_equal(a.tensor(5, 7), b.tensor(5, 7))
    g = a.tensor(1, 9, scale=0.02)
    e = b.gaussians_f32(1, 9, 0.02)
    assert np.array_equal(g, e)
