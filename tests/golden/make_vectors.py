"""Writes the golden vectors of this folder (``sb_*.npz``).  Run: python tests/golden/make_vectors.py
(``python tests/golden/make_vectors.py overflow`` writes only ``sb_packed_overflow.npz``,
``python tests/golden/make_vectors.py d256`` only ``sbdir_dense_d256.npz``)

The reference ships no fixtures for stick-breaking attention, so these come from the
mathematics alone, evaluated with 50-digit arithmetic (mpmath) and sharing no code with the
oracle or the kernels:

* forward: the product formula itself, term by term --
  beta_ij = 1 / (1 + exp(-s q_i.k_j)),  A_ij = beta_ij * prod_{j<k<i} (1 - beta_ik),
  o_i = sum_j A_ij v_j,  rem_i = prod_j (1 - beta_ij)   over the keys j that query i may see
  (j < i, or j <= i with attend_current);
* gradients: central differences of  loss = sum(o * dO) + sum(rem * dRem)  with a step of
  1e-20 at 50 digits (truncation error ~1e-40), one input element at a time.

The inputs are rounded to bfloat16-representable values, so the fp32 and the bf16 operator
read them without loss.  Each ``sb_*`` file holds float64 arrays q, k, v, do, drem, o, rem, dq, dk, dv in the
operator's layout ([B,H,T,D] dense, [H,sumT,D] packed), `scale`, `attend_current`, and for
the packed cases `cu_seqlens` (leading 0).  The ``sbdir_*`` files cover shapes of the
matrix-core kernels with directional derivatives in place of full gradients (see
run_directional_case); their inputs and directions are stored as float32, which holds them
exactly.
"""
import os

import numpy as np
from mpmath import mp, mpf, exp, fdot

mp.dps = 50
HERE = os.path.dirname(os.path.abspath(__file__))


def forward_one(q, k, v, scale, attend_current):
    """q, k, v: lists [T][D] of mpf for ONE (document, head).  Returns o [T][D], rem [T]."""
    T, D = len(q), len(q[0])
    o = [[mpf(0)] * D for _ in range(T)]
    rem = [mpf(1)] * T
    for i in range(T):
        last = i if attend_current else i - 1
        stick = mpf(1)                      # prod of (1 - beta_ik) over the keys right of j
        for j in range(last, -1, -1):
            z = scale * fdot(q[i], k[j])
            beta = 1 / (1 + exp(-z))
            a = beta * stick
            for c in range(D):
                o[i][c] += a * v[j][c]
            stick *= 1 - beta
        rem[i] = stick
    return o, rem


def loss_one(q, k, v, do, drem, scale, attend_current):
    o, rem = forward_one(q, k, v, scale, attend_current)
    T, D = len(q), len(q[0])
    return sum(fdot(o[i], do[i]) for i in range(T)) + fdot(rem, drem)


def grads_one(q, k, v, do, drem, scale, attend_current):
    h = mpf(10) ** -20
    out = []
    for which in range(3):
        src = (q, k, v)[which]
        g = [[mpf(0)] * len(src[0]) for _ in range(len(src))]
        for t in range(len(src)):
            for c in range(len(src[0])):
                keep = src[t][c]
                vals = []
                for sign in (1, -1):
                    src[t][c] = keep + sign * h
                    vals.append(loss_one(q, k, v, do, drem, scale, attend_current))
                src[t][c] = keep
                g[t][c] = (vals[0] - vals[1]) / (2 * h)
        out.append(g)
    return out


def bf16_exact(a):
    """Rounds to the nearest bfloat16 (ties to even), so that fp32 and bf16 operators read
    exactly the inputs the vectors were computed from."""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def to_mp(a):
    return [[mpf(float(x)) for x in row] for row in a]


def run_case(name, rng, H, lens, D, scale, attend_current, in_scale, packed):
    """One batch row (dense: lens = [T]) or a pack of documents."""
    total = sum(lens)
    q, k, v, do = (rng.standard_normal((H, total, D)) for _ in range(4))
    q, k, v, do, drem = (bf16_exact(x) for x in (q * in_scale, k * in_scale, v, do, rng.standard_normal((H, total))))
    res = {n: np.zeros((H, total, D)) for n in ("o", "dq", "dk", "dv")}
    rem = np.zeros((H, total))
    start = 0
    for L in lens:
        sl = slice(start, start + L)
        for h in range(H):
            args = [to_mp(x[h, sl]) for x in (q, k, v, do)] + [[mpf(float(x)) for x in drem[h, sl]]]
            o_, rem_ = forward_one(args[0], args[1], args[2], mpf(scale), attend_current)
            dq_, dk_, dv_ = grads_one(*args, mpf(scale), attend_current)
            res["o"][h, sl] = np.array(o_, dtype=np.float64).reshape(L, D)
            rem[h, sl] = np.array(rem_, dtype=np.float64)
            for n, g in (("dq", dq_), ("dk", dk_), ("dv", dv_)):
                res[n][h, sl] = np.array(g, dtype=np.float64).reshape(L, D)
        start += L
    arrays = dict(q=q, k=k, v=v, do=do, drem=drem, rem=rem, **res)
    if packed:
        arrays["cu_seqlens"] = np.cumsum([0] + list(lens)).astype(np.int32)
    else:                                     # [H,T,..] -> [B=1,H,T,..]
        arrays = {n: a[None] for n, a in arrays.items()}
    arrays["scale"] = np.float64(scale)
    arrays["attend_current"] = np.bool_(attend_current)
    np.savez(os.path.join(HERE, name + ".npz"), **arrays)
    print(name, "written", flush=True)


def run_directional_case(name, rng, lens, D, scale, attend_current, in_scale, packed, n_dirs=3):
    """Shapes the matrix-core kernels take (D = 64 or 128, more than one 128-row block), one
    head: the full o and rem, and -- a central difference per input element being out of
    reach here -- directional derivatives: for each random direction u of q (k, v), the
    derivative of the loss along u, which equals <dq, u> (<dk, u>, <dv, u>)."""
    total = sum(lens)
    q, k, v, do = (rng.standard_normal((total, D)) for _ in range(4))
    q, k, v, do, drem = (bf16_exact(x) for x in (q * in_scale, k * in_scale, v, do, rng.standard_normal(total)))
    dirs = bf16_exact(rng.standard_normal((3, n_dirs, total, D)))
    o, rem, slopes = np.zeros((total, D)), np.zeros(total), np.zeros((3, n_dirs))
    h = mpf(10) ** -20
    start = 0
    for L in lens:
        sl = slice(start, start + L)
        base = [to_mp(x[sl]) for x in (q, k, v, do)] + [[mpf(float(x)) for x in drem[sl]]]
        o_, rem_ = forward_one(base[0], base[1], base[2], mpf(scale), attend_current)
        o[sl] = np.array(o_, dtype=np.float64).reshape(L, D)
        rem[sl] = np.array(rem_, dtype=np.float64)
        for which in range(3):
            for n in range(n_dirs):
                u = to_mp(dirs[which, n, sl])
                vals = []
                for sign in (1, -1):
                    moved = list(base)
                    moved[which] = [[x + sign * h * d for x, d in zip(row, urow)] for row, urow in zip(base[which], u)]
                    vals.append(loss_one(*moved, mpf(scale), attend_current))
                slopes[which, n] += float((vals[0] - vals[1]) / (2 * h))   # documents add up
                print(name, "doc", start, "input", which, "direction", n, flush=True)
        start += L
    arrays = dict(q=q[None], k=k[None], v=v[None], do=do[None], drem=drem[None], o=o[None], rem=rem[None])
    if packed:
        arrays["cu_seqlens"] = np.cumsum([0] + list(lens)).astype(np.int32)
    else:
        arrays = {n: a[None] for n, a in arrays.items()}
    arrays = {n: a.astype(np.float32) if n in ("q", "k", "v", "do", "drem") else a for n, a in arrays.items()}   # bf16-exact
    arrays.update(directions=dirs.astype(np.float32), slopes=slopes, scale=np.float64(scale), attend_current=np.bool_(attend_current))
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    print(name, "written", flush=True)


def run_overflow_case(name):
    """A packed batch whose second document holds, inside the 32 keys that one lane of the
    matrix-core kernels chains over, logits of +90 (the running product of 1 + e^z leaves the
    fp32 range) followed further left by logits of -200 (e^z is exactly 0 in fp32) and by the keys
    of the previous document and of the diagonal, which are masked: a chain kept as that product
    meets inf * 0 there.  Own random stream, so that adding it does not move the other cases."""
    rng = np.random.default_rng(20250117)
    lens, D, H = [5, 40], 4, 1
    total = sum(lens)
    q, k, v, do = (rng.standard_normal((H, total, D)) * s for s in (0.5, 0.5, 1.0, 1.0))
    q[0, 25:, :] = 0.0
    q[0, 25:, 1] = 4.0                     # queries 20.. of the second document look along one coordinate
    k[0, 17:21, :] = 0.0
    k[0, 17:21, 1] = 45.0                  # logit +90 at scale 0.5
    k[0, 9:13, :] = 0.0
    k[0, 9:13, 1] = -100.0                 # logit -200
    q, k, v, do, drem = (bf16_exact(x) for x in (q, k, v, do, rng.standard_normal((H, total))))
    scale, attend_current = 0.5, False
    res = {n: np.zeros((H, total, D)) for n in ("o", "dq", "dk", "dv")}
    rem = np.zeros((H, total))
    start = 0
    for L in lens:
        sl = slice(start, start + L)
        args = [to_mp(x[0, sl]) for x in (q, k, v, do)] + [[mpf(float(x)) for x in drem[0, sl]]]
        o_, rem_ = forward_one(args[0], args[1], args[2], mpf(scale), attend_current)
        dq_, dk_, dv_ = grads_one(*args, mpf(scale), attend_current)
        res["o"][0, sl] = np.array(o_, dtype=np.float64).reshape(L, D)
        rem[0, sl] = np.array(rem_, dtype=np.float64)
        for n, g in (("dq", dq_), ("dk", dk_), ("dv", dv_)):
            res[n][0, sl] = np.array(g, dtype=np.float64).reshape(L, D)
        start += L
    arrays = dict(q=q, k=k, v=v, do=do, drem=drem, rem=rem, **res)
    arrays["cu_seqlens"] = np.cumsum([0] + list(lens)).astype(np.int32)
    arrays["scale"] = np.float64(scale)
    arrays["attend_current"] = np.bool_(attend_current)
    np.savez(os.path.join(HERE, name + ".npz"), **arrays)
    print(name, "written", flush=True)


if __name__ == "__main__":
    import sys
    if sys.argv[1:] == ["overflow"]:       # only the case added last
        run_overflow_case("sb_packed_overflow")
        sys.exit(0)
    if sys.argv[1:] == ["d256"]:           # head_dim 256, added later: a generator of its own leaves the other files as they are
        run_directional_case("sbdir_dense_d256", np.random.default_rng(20250311), lens=[150], D=256, scale=1 / 16.0,
                             attend_current=False, in_scale=1.0, packed=False)
        sys.exit(0)
    rng = np.random.default_rng(20240607)
    run_case("sb_dense_strict", rng, H=2, lens=[9], D=4, scale=0.7, attend_current=False, in_scale=1.0, packed=False)
    run_case("sb_dense_current", rng, H=2, lens=[6], D=3, scale=3 ** -0.5, attend_current=True, in_scale=1.0, packed=False)
    # logits out to about +-40: exercises the saturated branches of sigmoid / softplus
    run_case("sb_dense_saturated", rng, H=1, lens=[7], D=2, scale=1.0, attend_current=False, in_scale=4.0, packed=False)
    run_case("sb_packed_strict", rng, H=2, lens=[4, 1, 7], D=4, scale=0.5, attend_current=False, in_scale=1.0, packed=True)
    run_case("sb_packed_current", rng, H=2, lens=[3, 5], D=4, scale=0.5, attend_current=True, in_scale=1.5, packed=True)
    # matrix-core shapes (minutes of 50-digit arithmetic)
    run_directional_case("sbdir_dense_d64", rng, lens=[150], D=64, scale=0.125, attend_current=False, in_scale=1.0, packed=False)
    run_directional_case("sbdir_packed_d64", rng, lens=[40, 136], D=64, scale=0.125, attend_current=True, in_scale=1.0, packed=True)
    run_directional_case("sbdir_dense_d128", rng, lens=[130], D=128, scale=128 ** -0.5, attend_current=True, in_scale=1.0, packed=False)
    run_overflow_case("sb_packed_overflow")
