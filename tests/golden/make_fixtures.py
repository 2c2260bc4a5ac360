"""Writes the golden fixtures of this folder: inputs and expected outputs of the fused
convolution (forward and VJP) for four small cases, as `.npz` files.

    python tests/golden/make_fixtures.py

The reference implementation cannot run here (no JAX), so the expected values come from this
repository's float64 CPU restatement (`oracle/conv_oracle.py`), which is itself pinned by the
closed-form strip case of `lib/e3j_ops/tests/test_convolution.cpp:122-207`, by loop restatements
of the reference's CPU checkers and by autograd / finite differences (`tests/test_oracle.py`).
The fixtures freeze those values: a later change of the oracle, of the table construction or of
the kernels shows up as a difference to a file that is under version control.

Cases:
  strip            the reference's hand-computable case (4 nodes, 6 edges, table of ones); the
                   expected forward is the closed form, exact in float32
  l3_k64           16 nodes, 48 edges, the 0e+1o+2e+3o x lmax 3 -> l<=3 table, 64 channels
                   (the table the 1M-edge configuration uses; runs the unrolled kernels)
  padding          dummy senders / receivers (INT32_MAX) at the tail, an isolated node, a
                   random table with an uncovered output row and path
  unsorted_skewed  edges in random order with one hub node, `GraphOrdering.NONE`
Arrays are in the trailing-channels layout; expected values are float64 except in `l3_k64`
(float32 and no `mag_*`, to keep the file small: compare at 1e-6 relative there).  `mag_*` are the sums of the absolute values of the
terms of every expected element, which bound the float32 summation-order noise.
"""

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import conv_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
DUMMY = np.iinfo(np.int32).max


def expected(idx, val, mix, x, y, s, snd, rcv, dm, num_out):
    def both(v, xs, ys, ss, dms):
        out = O.convolution_unfused(idx, v, mix, xs, ys, ss, snd, rcv, num_out, dtype=np.float64)
        dx, dy, ds = O.convolution_vjp(idx, v, mix, xs, ys, ss, snd, rcv, dms, dtype=np.float64)
        return out, dx, dy, ds
    out, dx, dy, ds = both(val, x, y, s, dm)
    m_out, m_dx, m_dy, m_ds = both(np.abs(val), np.abs(x), np.abs(y), np.abs(s), np.abs(dm))
    return dict(out=out, dx=dx, dy=dy, ds=ds, mag_out=m_out, mag_dx=m_dx, mag_dy=m_dy, mag_ds=m_ds)


def save(name, **arrays):
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **arrays)
    print(f"{path}: {os.path.getsize(path) / 1024:.0f} KiB")


def random_table(rng, nnz, X, Y, Z, S, skip_row=None, skip_path=None):
    """Unique (i, j, k) triples with normal values; one scalar per output row."""
    rows = [i for i in range(Z) if i != skip_row]
    paths = [l for l in range(S) if l != skip_path]
    mix = np.zeros(Z, dtype=np.int64)
    for n, i in enumerate(range(Z)):
        mix[i] = paths[n % len(paths)]
    triples = set()
    while len(triples) < nnz:
        triples.add((rows[rng.integers(len(rows))], int(rng.integers(X)), int(rng.integers(Y))))
    idx = np.array(sorted(triples), dtype=np.int64)
    val = rng.standard_normal(len(idx)).astype(np.float32)
    return idx, val, mix


def main():
    # 1. strip case --------------------------------------------------------------------------
    c = O.strip_case(num_strips=3, channels=32, scale_s=True)
    rng = np.random.default_rng(100)
    dm = rng.integers(-3, 4, size=c["expect"].shape).astype(np.float32)  # small integers: exact sums
    e = expected(c["idx"], c["val"], c["mix_idx"], c["x"], c["y"], c["s"], c["sender"], c["receiver"],
                 dm, c["num_out"])
    assert np.array_equal(e["out"], c["expect"].astype(np.float64))
    save("strip", idx=c["idx"], val=c["val"], mix=c["mix_idx"], x=c["x"], y=c["y"], s=c["s"],
         sender=c["sender"], receiver=c["receiver"], dm=dm, num_nodes=4, num_out=c["num_out"],
         num_scalars=3, ordering="RECEIVER", **e)

    # 2. the l<=3 table at 64 channels ---------------------------------------------------------
    from e3j_amd import Convolution
    m = Convolution(("0e+1o+2e+3o", "0e+1o+2e+3o"), "0e+1o+2e+3o", graph_ordering="RECEIVER")
    coef = m.coef
    idx = np.asarray(coef.idx, dtype=np.int64)[:, :3]
    val = np.asarray(coef.val, dtype=np.float32)
    mix = np.asarray(m._mix.mix_indices, dtype=np.int64)
    rng = np.random.default_rng(101)
    N, E, K = 16, 48, 64
    rcv = np.sort(rng.integers(0, N, size=E)).astype(np.int32)
    snd = rng.integers(0, N, size=E).astype(np.int32)
    x = rng.standard_normal((N, 16, K)).astype(np.float32)
    y = rng.standard_normal((E, 16)).astype(np.float32)
    s = (rng.standard_normal((E, 23, K)) * 0.5).astype(np.float32)
    dm = rng.standard_normal((N, 99, K)).astype(np.float32)
    e = expected(idx, val, mix, x, y, s, snd, rcv, dm, 99)
    save("l3_k64", idx=idx, val=val, mix=mix, x=x, y=y, s=s, sender=snd, receiver=rcv, dm=dm,
         num_nodes=N, num_out=99, num_scalars=23, ordering="RECEIVER",
         **{k: v.astype(np.float32) for k, v in e.items() if not k.startswith("mag")})  # small file

    # 3. padding edges, isolated node, uncovered row and path ----------------------------------
    rng = np.random.default_rng(102)
    N, E, K, X, Y, Z, S = 9, 40, 20, 5, 6, 8, 4
    idx, val, mix = random_table(rng, 70, X, Y, Z, S, skip_row=3, skip_path=2)
    live = 33
    rcv = np.sort(rng.choice([n for n in range(N - 1) if n != 4], size=live)).astype(np.int32)  # node 4 isolated
    snd = rng.integers(0, N - 1, size=live).astype(np.int32)
    snd = np.concatenate([snd, [DUMMY, 2, DUMMY, DUMMY, 1, DUMMY, DUMMY]]).astype(np.int32)
    rcv = np.concatenate([rcv, [DUMMY, DUMMY, DUMMY, DUMMY, DUMMY, DUMMY, DUMMY]]).astype(np.int32)
    x = rng.standard_normal((N, X, K)).astype(np.float32)
    y = rng.standard_normal((E, Y)).astype(np.float32)
    s = rng.standard_normal((E, S, K)).astype(np.float32)
    dm = rng.standard_normal((N, Z, K)).astype(np.float32)
    e = expected(idx, val, mix, x, y, s, snd, rcv, dm, Z)
    assert not e["out"][4].any() and not e["out"][:, 3].any() and not e["ds"][live:].any()
    save("padding", idx=idx, val=val, mix=mix, x=x, y=y, s=s, sender=snd, receiver=rcv, dm=dm,
         num_nodes=N, num_out=Z, num_scalars=S, ordering="RECEIVER", **e)

    # 4. unsorted edges, one hub ------------------------------------------------------------------
    rng = np.random.default_rng(103)
    N, K, X, Y, Z, S = 24, 16, 4, 9, 7, 3
    idx, val, mix = random_table(rng, 90, X, Y, Z, S)
    rcv = np.concatenate([np.full(60, 5), rng.integers(0, N, size=100)]).astype(np.int32)
    snd = rng.integers(0, N, size=rcv.size).astype(np.int32)
    shuffle = rng.permutation(rcv.size)
    rcv, snd = rcv[shuffle], snd[shuffle]
    E = rcv.size
    x = rng.standard_normal((N, X, K)).astype(np.float32)
    y = rng.standard_normal((E, Y)).astype(np.float32)
    s = rng.standard_normal((E, S, K)).astype(np.float32)
    dm = rng.standard_normal((N, Z, K)).astype(np.float32)
    e = expected(idx, val, mix, x, y, s, snd, rcv, dm, Z)
    save("unsorted_skewed", idx=idx, val=val, mix=mix, x=x, y=y, s=s, sender=snd, receiver=rcv, dm=dm,
         num_nodes=N, num_out=Z, num_scalars=S, ordering="NONE", **e)


if __name__ == "__main__":
    main()
