"""Writes tests/golden/mwc_kat.json: known answers of the multiply-with-carry
generator computed with the Python-integer coding in oracle/mwc.py (not with the
numpy or C codings the tests then compare against them).

The reference ships no RNG vectors and cannot be built or imported here, so these
are answers of the restated recurrence (cudamat/cudamat_kernels.cu:96-123), kept
as a regression pin for all three codings and for the device.

Run from the repository root:  python tests/golden/make_mwc_kat.py
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import mwc  # noqa: E402

MULTS = mwc.load_multipliers(os.path.join(ROOT, 'deepnet_amd', 'rnd_multipliers_32bit.txt'))


def main():
    kat = {'multipliers_md5': hashlib.md5(open(os.path.join(ROOT, 'deepnet_amd', 'rnd_multipliers_32bit.txt'),
                                               'rb').read()).hexdigest(),
           'streams': {}}
    for seed in (0, 1, 42):
        for stream in (0, 1, 12287):
            mult = int(MULTS[stream])
            w = mwc.seed_word_py(seed, mult)
            entry = {'mult': mult, 'seeded_word': w, 'draw_words': [], 'draw_uniform_bits': []}
            for _ in range(4):
                w = mwc.step_py(w, mult)
                entry['draw_words'].append(w)
                entry['draw_uniform_bits'].append(int(np.float32(mwc.uniform_py(w)).view(np.uint32)))
            kat['streams']['%d:%d' % (seed, stream)] = entry
    # one whole call of 3*12288+5 elements, seed 42, as a digest of the float32 bytes
    n = 3 * mwc.NUM_RND_STREAMS + 5
    words = [mwc.seed_word_py(42, int(m)) for m in MULTS]
    out = np.empty(n, dtype=np.float32)
    for i in range(n):
        t = i % mwc.NUM_RND_STREAMS
        words[t] = mwc.step_py(words[t], int(MULTS[t]))
        out[i] = mwc.uniform_py(words[t])
    kat['fill_seed42'] = {'n': n, 'sha256': hashlib.sha256(out.tobytes()).hexdigest(),
                          'first8_bits': [int(v) for v in out[:8].view(np.uint32)],
                          'last8_bits': [int(v) for v in out[-8:].view(np.uint32)],
                          'state_sha256': hashlib.sha256(np.array(words, dtype=np.uint64).tobytes()).hexdigest()}
    with open(os.path.join(ROOT, 'tests', 'golden', 'mwc_kat.json'), 'w') as f:
        json.dump(kat, f, indent=1)
    print("wrote mwc_kat.json")


if __name__ == '__main__':
    main()
