#!/usr/bin/env python3
"""Writes tests/golden/brute_force_cases.npz: small CTC-Transducer lattices
with their log-likelihood and the dense gradient of the cost, obtained by
enumerating every alignment (tests/ctct_cases.py: brute_force) in float64.

Nothing of the reference implementation is imported or run: the reference
ships no golden vectors or tests of its own (its only demo, ref_ctct.py:233-255,
prints values without recording any), so these vectors come from the
definition of the loss (README.md:4-13 of the reference: every frame emits
blank, a repeat of the current label, or the next label; the score of a frame
is read at the context of labels started before it).

    python tests/golden/make_brute_force_fixtures.py

The batch is padded to (N, T, U+1, V) with zeros outside lx / ly, like the
inputs of the GPU tests.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from ctct_cases import brute_force, log_softmax   # noqa: E402

# labels, frames, vocabulary, scale of the logits
CASES = [
    ([1], 1, 3, 1.0),
    ([1], 4, 3, 1.0),
    ([1, 2], 5, 4, 1.0),
    ([2, 2], 5, 4, 1.0),          # a repeated label needs a blank between
    ([1, 1, 2], 6, 3, 2.0),
    ([3, 1, 3], 7, 5, 1.0),
    ([2, 1, 1], 4, 3, 1.0),       # lx = ly + repeats: a single alignment skeleton
    ([], 3, 4, 1.0),              # no labels: blanks only
    ([1, 2, 3], 3, 4, 3.0),       # lx = ly: one alignment
]


def main():
    rng = np.random.default_rng(20240607)
    N = len(CASES)
    T = max(c[1] for c in CASES)
    U = max(len(c[0]) for c in CASES)
    V = max(c[2] for c in CASES)
    joint = np.zeros((N, T, U + 1, V), np.float64)
    dense = np.zeros_like(joint)
    ys = np.zeros((N, U), np.int32)
    lx = np.zeros(N, np.int32)
    ly = np.zeros(N, np.int32)
    loglik = np.zeros(N, np.float64)
    for n, (labels, frames, vocab, sigma) in enumerate(CASES):
        u1 = len(labels) + 1
        lp = log_softmax(rng.standard_normal((frames, u1, vocab)) * sigma)
        # the kernels read float32 inputs: enumerate on the rounded values
        lp = lp.astype(np.float32).astype(np.float64)
        ll, d = brute_force(lp, labels)
        joint[n, :frames, :u1, :vocab] = lp
        # columns beyond this case's vocabulary never occur in its labels; give
        # them a finite log-probability so that the padded batch is a valid input
        joint[n, :frames, :u1, vocab:] = -30.0
        dense[n, :frames, :u1, :vocab] = d
        ys[n, :len(labels)] = labels
        lx[n], ly[n] = frames, len(labels)
        loglik[n] = ll
    out = os.path.join(HERE, "brute_force_cases.npz")
    np.savez_compressed(out, joint=joint.astype(np.float32), ys=ys, lx=lx, ly=ly, loglik=loglik,
                        dense_grad=dense)
    print("wrote", out, os.path.getsize(out), "bytes; costs", -loglik)


if __name__ == "__main__":
    main()
