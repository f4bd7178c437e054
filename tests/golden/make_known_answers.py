"""Writes the golden vectors under tests/golden/ by running the reference's own
host header (HiPC18/src/util.h, compiled as it lies by oracle/Makefile into
oracle/_ref/libref_util.so).  Needs /root/reference; run once in the build
container:  python tests/golden/make_known_answers.py
The fixtures are data only (inputs and the outputs the reference produced)."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle  # noqa: E402


def main():
    assert oracle.have_ref(), "build oracle/_ref first (make -C oracle)"
    n_rows, n_cols, ts, actv = 4, 5, 2, 2
    rows, cols, vals = [0, 0, 1, 3, 3, 3], [0, 3, 2, 0, 1, 4], [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    rp, holder, nh = oracle.ref_make_csr(rows, cols, vals, n_rows)
    r, _ = oracle.ref_rewrite_1d(n_rows, n_cols, rows, cols, vals, ts, actv)
    ka = dict(n_rows=n_rows, n_cols=n_cols, rows=rows, cols=cols, vals=vals, tile_size_x=ts, actv_row_size=actv,
              row_ptr=rp[: nh + 1].tolist(), row_holder=holder[:nh].tolist(), ntile_c=r["n_tiles"],
              tiled_rows=r["t_rows"].tolist(), tiled_cols=r["t_cols"].tolist(), tiled_vals=r["t_vals"].tolist(),
              tiled_ind=r["tiled_ind"].tolist(), lastIdx_tile=r["last_idx_tile"].tolist(),
              active_row=[a.tolist() for a in r["active_row"]], n_actv_row=r["n_actv_row"].tolist(),
              first_block_end=[int(b[0]) for b in r["last_idx_block"]], max_active_row=r["max_active_rows"])
    json.dump(ka, open(os.path.join(HERE, "tiling_known_answer.json"), "w"), indent=1)
    X = oracle.ref_initial(1, 8)
    json.dump(dict(first8=[float(np.float32(x)) for x in X.ravel()]), open(os.path.join(HERE, "initial_known_answer.json"), "w"), indent=1)


if __name__ == "__main__":
    main()
