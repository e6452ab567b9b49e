"""Writes tests/golden/qsa_soak_cases.npz: the selection lists of the QSA sparse attention cases
that a randomised parity soak found over the per-channel bound.

The soak drew every case from one numpy Generator stream, so a case is identified by the stream's
seed and its position in it; this script replays the draws (no GPU, no oracle call) up to each
wanted case and stores what the stream produced for it: the per-token lists of selected 4-token
groups, the counts, the token positions and the token mask.  Pool contents, queries and gates
come from the oracle's own seeded generators at test time (tests/cases.py), keyed by `seed`.

    python tests/golden/make_qsa_soak_cases.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from cases import make_case, qsa_groups_of  # noqa: E402
from oracle import DT_F16, FMT_FP16, FMT_FP8, FMT_Q8_0, FMT_TQ4, XF_IDENTITY, XF_WHT256  # noqa: E402

# (stream seed, case seed) of the cases over the bound
WANTED = {9: [678757, 163764, 813105], 772: [394998]}


def replay(stream_seed, wanted, limit=20000):
    rng = np.random.default_rng(stream_seed)
    found = {}
    for _ in range(limit):
        fmt = int(rng.choice([FMT_TQ4, FMT_TQ4, FMT_FP16, FMT_FP8, FMT_Q8_0]))
        xf = XF_WHT256 if fmt == FMT_TQ4 else (
            int(rng.choice([XF_IDENTITY, XF_WHT256])) if fmt in (FMT_FP8, FMT_Q8_0) else XF_IDENTITY)
        bs = int(rng.choice([16, 32, 64]))
        kvh = int(rng.choice([1, 2]))
        gqa = int(rng.choice([1, 2, 4, 6, 8]))
        seq_len = int(rng.integers(5, 3000))
        n_tok = int(rng.integers(1, 40))
        select_k = int(rng.choice([1, 3, 8, 33, 64, 129, 300]))
        seed = int(rng.integers(1, 1 << 20))
        n_groups = (seq_len + 3) // 4
        picks, kks, drops, nums, poss = [], [], [], [], []
        for _t in range(n_tok):
            kk = int(rng.integers(0, min(select_k, n_groups) + 1))
            picks.append(rng.permutation(n_groups)[:kk])
            drops.append([rng.random() < 0.05 for _j in range(kk)])
            kks.append(kk)
            nums.append(kk if rng.random() < 0.8 else int(rng.integers(0, select_k + 3)))
            poss.append(int(rng.integers(0, seq_len)))
        has_gate = bool(rng.random() < 0.6)
        mask = (rng.random(n_tok) > 0.15).astype(np.uint8) if rng.random() < 0.4 else None
        had = bool(rng.random() < 0.4)
        scratch = int(rng.choice([0, 4096, 16 << 20]))
        if seed in wanted:
            _pool, bt, _k, _v, _q, _aq, _ctx = make_case(fmt, bs, [seq_len], [1], seed, DT_F16, kv_heads=kvh, xf=xf)
            all_phys, all_log, _ = qsa_groups_of(bt, [seq_len], bs, select_k=n_groups)
            sel_phys = np.full((n_tok, select_k), -1, dtype=np.int32)
            sel_log = np.zeros((n_tok, select_k), dtype=np.int32)
            for t in range(n_tok):
                sel_phys[t, :kks[t]] = all_phys[0, picks[t]]
                sel_log[t, :kks[t]] = all_log[0, picks[t]]
                for j in range(kks[t]):
                    if drops[t][j]:
                        sel_phys[t, j] = -1
            found[seed] = dict(
                meta=np.array([fmt, xf, bs, kvh, gqa, seq_len, n_tok, select_k, int(has_gate), int(had), scratch, seed],
                              dtype=np.int64),
                sel_phys=sel_phys, sel_log=sel_log, num_sel=np.array(nums, dtype=np.int32),
                seq_pos=np.array(poss, dtype=np.int32),
                mask=mask if mask is not None else np.zeros(0, dtype=np.uint8))
            if len(found) == len(wanted):
                break
    return found


def main():
    out = {}
    for stream_seed, wanted in WANTED.items():
        found = replay(stream_seed, set(wanted))
        missing = set(wanted) - set(found)
        assert not missing, "stream %d: cases %s not reached" % (stream_seed, sorted(missing))
        for seed, d in found.items():
            for k, v in d.items():
                out["s%d_%s" % (seed, k)] = v
    np.savez_compressed(os.path.join(HERE, "qsa_soak_cases.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
