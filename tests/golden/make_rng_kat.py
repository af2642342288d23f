"""Writes rng_kat.npz: the first 16 draws of three streams of the library's seeded generator
(SplitMix64-keyed counter -> 24-bit uniform / Box-Muller normal / modulo integer).  A regression pin of
this build's own generator; the reference's RNG stream cannot be reproduced (its rng crate is not in its tree)."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from rembrandt_amd import synth  # noqa: E402

np.savez(os.path.join(os.path.dirname(os.path.abspath(__file__)), "rng_kat.npz"),
         normal=synth.normal(0x5EED0004, 100, (16,)), uniform=synth.uniform(0x5EED0001, 100, (16,)),
         integers=synth.integers(0x5EED0004, 200, (16,), 1000))
