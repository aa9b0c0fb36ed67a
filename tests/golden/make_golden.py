"""Writes the fixtures of this folder from the oracle (run from the repository root:
`python tests/golden/make_golden.py`).  They freeze the function the oracle computes today -- tables, paths
and samples of one small graph, and the table of the 40-entry toy row of the reference's test/tmp.cu:30-52 --
so that a later change of the oracle (or of the kernels checked against it) that moves a single bit shows up.
The Philox vectors are the published Random123 known answers, not oracle output."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import orc  # noqa: E402

SCALE, EF, SEED = 8, 8, 7
N, LEN = 64, 10
P, Q = 2.0, 0.5
FANOUT = [1, 4, 3]


def main():
    kat = [
        {"ctr": [0, 0, 0, 0], "key": [0, 0], "out": [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]},
        {"ctr": [0xffffffff] * 4, "key": [0xffffffff] * 2, "out": [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]},
        {"ctr": [0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], "key": [0xa4093822, 0x299f31d0],
         "out": [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]},
    ]
    with open(os.path.join(HERE, "philox_kat.json"), "w") as f:
        json.dump(kat, f, indent=1)

    toy_w = np.array([0.5] * 35 + [2.0] * 5, np.float32)
    toy_prob, toy_alias, _ = orc.alias_build_row(toy_w)
    np.savez_compressed(os.path.join(HERE, "toy_row.npz"), w=toy_w, prob=toy_prob, alias=toy_alias)

    xadj, adjncy = orc.rmat_csr(SCALE, EF, SEED)
    w = orc.gen_weights(orc.W_LOGNORMAL, SEED, len(adjncy), 0.0, 1.0)
    w[xadj[3]:xadj[4]] = 0.0  # one row of zero total weight
    prob, alias, valid = orc.alias_build(xadj, w)
    seeds = orc.gen_seeds(SEED, len(xadj) - 1, N)
    seeds[5] = len(xadj) + 10  # a start vertex that does not exist
    out = dict(xadj=xadj, adjncy=adjncy, w=w, prob=prob, alias=alias, valid=valid, seeds=seeds)
    out["dw_paths"], out["dw_lengths"], _ = orc.walk_offline(xadj, adjncy, prob, alias, seeds, LEN, 0.0, SEED)
    out["ppr_paths"], out["ppr_lengths"], _ = orc.walk_offline(xadj, adjncy, prob, alias, seeds, LEN, 0.15, SEED)
    out["n2v_paths"], out["n2v_lengths"], _ = orc.walk_online(xadj, adjncy, w, 1, P, Q, seeds, LEN, 0.0, SEED)
    out["rej_paths"], out["rej_lengths"], _ = orc.walk_node2vec_reject(xadj, adjncy, prob, alias, P, Q, seeds, LEN, 0.0,
                                                                      SEED)
    out["sample_data"], out["sample_lengths"], _ = orc.sample_offline(xadj, adjncy, prob, alias, seeds, FANOUT, SEED)
    np.savez_compressed(os.path.join(HERE, "rmat_s8.npz"), **out)
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
