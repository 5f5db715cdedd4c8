"""Writes the golden vectors under tests/golden/ from the reference's own CPU path.

Run in the build container only (needs /root/reference and oracle/_ref, built by
`make -C oracle ref`).  For every case the seeded fp16 score tensor is handed to
the compiled reference (`openfish_decode_cpu`, -DDEBUG build so that it also
dumps its bwd/fwd/post/qual_data/base_probs/total_probs tensors) and inputs and
outputs are stored in one compressed .npz.  The three output blobs and the
score blob of the reference's in-repo test (test/data/*.blob, fast model, N=1)
are copied alongside as ref_fixture_*.blob: they are data files of its test suite.
"""
import os
import shutil
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from openfish_amd import synth  # noqa: E402
from oracle import crf_oracle as O  # noqa: E402

REF_DATA = "/root/reference/test/data"

# name: (state_len, T, N, seed, stress, opt)
CASES = {
    "sl1_plain": (1, 48, 3, 11, False, {}),
    "sl2_plain": (2, 80, 3, 12, False, {}),
    "fast_plain": (3, 300, 4, 13, False, dict(q_scale=0.97, q_shift=-1.8)),
    "fast_stress": (3, 300, 4, 14, True, dict(q_scale=0.97, q_shift=-1.8)),
    "fast_cut5_blank1p5": (3, 200, 3, 15, False, dict(beam_cut=5.0, blank_score=1.5)),
    "hac_plain": (4, 160, 2, 16, False, dict(q_scale=0.95, q_shift=-0.2)),
    "hac_stress": (4, 160, 2, 17, True, dict(q_scale=0.95, q_shift=-0.2)),
    "sup_plain": (5, 64, 2, 18, False, dict(q_scale=0.95, q_shift=0.5)),
}


def main():
    assert O.have_ref(), "build oracle/_ref first: make -C oracle ref"
    for name, (sl, T, N, seed, stress, opt) in CASES.items():
        scale = synth.stress_scale(N) if stress else None
        s16 = synth.crf_scores(T, N, sl, seed=seed, chunk_scale=scale)
        full = O.default_opt(**opt)
        ref = O.ref_decode(s16.astype(np.float32), sl, full, nthreads=2, tensors=True)
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"), scores=s16, state_len=np.int32(sl),
            opt=np.array([full["beam_cut"], full["blank_score"], full["q_shift"], full["q_scale"]], np.float32),
            **ref)
        print(name, "T", T, "N", N, "bases", int(ref["moves"].sum()))
    for f in ("scores", "moves", "sequence", "qstring"):
        shutil.copyfile(os.path.join(REF_DATA, f + ".blob"), os.path.join(HERE, "ref_fixture_" + f + ".blob"))
        os.chmod(os.path.join(HERE, "ref_fixture_" + f + ".blob"), 0o644)


if __name__ == "__main__":
    main()
