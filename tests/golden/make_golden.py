"""Writes tests/golden/*.npz: inputs and expected outputs for the MoE expert path.

The expected values do NOT come from the oracle under ``oracle/`` (which these
fixtures are used to check) nor from the reference's Python: they are computed
here by independent means —

* ``worked_example``: the 3-token, top-2, 3-expert example, typed in by hand
  and re-derived below with Python's ``sorted`` on (expert, position) pairs;
* ``gmm_cases``: the shapes and group lists of the reference's own grouped-matmul
  unit test (tests_extend/unit_tests/ops/cann/test_npu_gmm.py:63-126) and doc
  example (docs/zh/ops/gmm.md:65-73), filled with small integers so that every
  product and partial sum is exact in bf16, fp16 and fp32 alike, multiplied
  with numpy int64 matmuls per group;
* ``groupmatmul_add``: the identity of
  tests_extend/unit_tests/ops/atb/test_groupmatmul_add.py:16-33 at reduced size,
  again on integers;
* ``layer_fp64``: the plumbing pipeline (permute, grouped matmul, SiLU*gate,
  grouped matmul, weighted unpermute; 8 experts, top-2) at 96 tokens, hidden 64,
  FFN 96, evaluated with explicit per-token numpy fp64 loops.

Run from the repo root: ``python tests/golden/make_golden.py``.
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def stable_order(flat):
    return np.array(sorted(range(len(flat)), key=lambda i: (int(flat[i]), i)), dtype=np.int64)


def worked_example():
    indices = np.array([[1, 0], [0, 2], [1, 2]], dtype=np.int64)
    flat = indices.reshape(-1)
    fwd = stable_order(flat)
    assert fwd.tolist() == [1, 2, 0, 4, 3, 5]          # typed-in expectation
    inv = np.empty_like(fwd)
    inv[fwd] = np.arange(len(fwd))
    assert inv.tolist() == [2, 0, 1, 4, 3, 5]
    tokens = np.arange(3 * 4, dtype=np.float32).reshape(3, 4) + 1.0
    permuted = tokens[fwd // 2]
    probs = np.array([[0.25, 0.75], [0.5, 0.5], [1.0, 0.0]], dtype=np.float32)
    out = np.zeros_like(tokens)
    for t in range(3):
        for j in range(2):
            out[t] += probs[t, j] * permuted[inv[t * 2 + j]]
    np.savez(os.path.join(HERE, "worked_example.npz"), indices=indices, tokens=tokens, sorted_indices=fwd,
             row_id_map=inv.astype(np.int32), permuted=permuted, probs=probs, unpermuted=out,
             tokens_per_expert=np.bincount(flat, minlength=3))


def int_matrix(rng, shape, lo=-3, hi=4):
    return rng.integers(lo, hi, size=shape).astype(np.int64)


def gmm_cases():
    rng = np.random.default_rng(20240611)
    out = {}
    # group_type 0 (split rows of x): x[M,K] @ w[E,K,N]
    for name, m, counts in (("rows_a", 32, [1, 2, 3, 4, 5, 6, 7, 4]), ("rows_b", 42, [1, 3, 5, 7, 9, 6, 7, 4]),
                            ("rows_doc", 32, [4] * 8)):
        k, n = (64, 32) if name != "rows_doc" else (256, 32)
        lim = 2 if k <= 64 else 1               # |y| <= k*lim*lim <= 256: exact even in bf16
        x = int_matrix(rng, (m, k), -lim, lim + 1)
        w = int_matrix(rng, (len(counts), k, n), -lim, lim + 1)
        y = np.zeros((m, n), dtype=np.int64)
        s = 0
        for g, c in enumerate(counts):
            y[s:s + c] = x[s:s + c] @ w[g]
            s += c
        out[f"{name}_x"], out[f"{name}_w"], out[f"{name}_y"] = x, w, y
        out[f"{name}_counts"] = np.array(counts, dtype=np.int64)
    # group_type 2 (split the reduction dim): x^T[48, M] @ w[M, 64] per group, incl. empty groups
    for name, m, counts in (("red_a", 32, [1, 2, 3, 4, 5, 6, 7, 4]), ("red_empty", 42, [9, 0, 0, 7, 9, 6, 7, 4])):
        x = int_matrix(rng, (m, 48))          # stored [M, 48]; the op sees x.T
        w = int_matrix(rng, (m, 64))
        y = np.zeros((len(counts), 48, 64), dtype=np.int64)
        s = 0
        for g, c in enumerate(counts):
            y[g] = x[s:s + c].T @ w[s:s + c]
            s += c
        out[f"{name}_x"], out[f"{name}_w"], out[f"{name}_y"] = x, w, y
        out[f"{name}_counts"] = np.array(counts, dtype=np.int64)
    np.savez_compressed(os.path.join(HERE, "gmm_cases.npz"), **{k: v.astype(np.int32) for k, v in out.items()})


def groupmatmul_add():
    rng = np.random.default_rng(7)
    x = int_matrix(rng, (96, 40), -2, 3)      # |x^T dy| <= 50*4: exact in bf16 too
    dy = int_matrix(rng, (96, 24), -2, 3)
    offsets = np.array([50, 96], dtype=np.int64)            # cumulative, as in the reference test
    acc = int_matrix(rng, (2 * 40, 24), -8, 9)
    expect = acc.copy().reshape(2, 40, 24)
    s = 0
    for g, e in enumerate(offsets):
        expect[g] += x[s:e].T @ dy[s:e]
        s = e
    np.savez_compressed(os.path.join(HERE, "groupmatmul_add.npz"), x=x.astype(np.int32), dy=dy.astype(np.int32),
                        offsets=offsets, acc=acc.astype(np.int32), expect=expect.reshape(2 * 40, 24).astype(np.int32))


def layer_fp64():
    rng = np.random.default_rng(0)
    T, H, E, K, F = 96, 64, 8, 2, 96
    x = rng.standard_normal((T, H))
    logits = rng.standard_normal((T, E))
    p_full = np.exp(logits - logits.max(-1, keepdims=True))
    p_full /= p_full.sum(-1, keepdims=True)
    idx = np.argsort(-p_full, axis=-1, kind="stable")[:, :K]
    p = np.take_along_axis(p_full, idx, -1)
    p /= p.sum(-1, keepdims=True)
    w1 = rng.standard_normal((E, H, 2 * F)) * 0.02
    w2 = rng.standard_normal((E, F, H)) * 0.02
    # the fixture stores fp32 inputs: evaluate on exactly those values, in fp64
    x, p, w1, w2 = (a.astype(np.float32).astype(np.float64) for a in (x, p, w1, w2))
    out = np.zeros((T, H))
    for t in range(T):
        for j in range(K):
            e = idx[t, j]
            h = x[t] @ w1[e]
            g, u = h[:F], h[F:]
            a = g / (1.0 + np.exp(-g)) * u
            out[t] += p[t, j] * (a @ w2[e])
    np.savez_compressed(os.path.join(HERE, "layer_fp64.npz"), x=x.astype(np.float32), idx=idx.astype(np.int64),
                        p=p.astype(np.float32), w1=w1.astype(np.float32), w2=w2.astype(np.float32), out=out)


if __name__ == "__main__":
    worked_example()
    gmm_cases()
    groupmatmul_add()
    layer_fp64()
    print("golden fixtures written to", HERE)
