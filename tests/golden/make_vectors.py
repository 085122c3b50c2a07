"""Writes tests/golden/attention_vectors.npz: small fixed inputs and their expected outputs, computed
here with scalar fp64 loops that state the operators' definitions directly (independent of oracle/ and
of the kernels).  The reference holds no fixtures of its own; these freeze the semantics the tests rely
on -- bottom-right causal alignment, rows without keys, grouped heads, the piecewise distance rule, the
paged block table -- so that a change to the oracle or the kernels that alters them is caught by fixed
numbers.  Inputs are fp16-representable, so every implementation starts from identical values.

    python tests/golden/make_vectors.py
"""
import math
import os

import numpy as np


def f16(rng, shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float16).astype(np.float64)


def flash(q, k, v, causal, sm_scale):
    """o, log-normalizer, total attention.  q (B, H, M, D), k/v (B, Hk, N, D); query head h uses kv head
    h // (H / Hk); key n is visible to query m iff not causal or m + (N - M) >= n; a row without visible
    keys gives o = 0, L = -inf."""
    B, H, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    o = np.zeros((B, H, M, D))
    L = np.full((B, H, M), -np.inf)
    tot = np.zeros((B, H, N))
    for b in range(B):
        for h in range(H):
            hk = h // (H // Hk)
            for m in range(M):
                vis = [n for n in range(N) if (not causal) or (m + N - M >= n)]
                if not vis:
                    continue
                s = [sm_scale * float(np.dot(q[b, h, m], k[b, hk, n])) for n in vis]
                top = max(s)
                e = [math.exp(x - top) for x in s]
                z = sum(e)
                L[b, h, m] = top + math.log(z)
                for n, en in zip(vis, e):
                    o[b, h, m] += (en / z) * v[b, hk, n]
                    tot[b, h, n] += en / z
    return o, L, tot


def piecewise(q1, k1, q2, k2, v, w, causal, sm_scale):
    """The score of (m, n) is q2.k2 when m + (N - M) - n >= w and q1.k1 otherwise."""
    B, H, M, D = q1.shape
    N = k1.shape[2]
    o = np.zeros((B, H, M, D))
    for b in range(B):
        for h in range(H):
            for m in range(M):
                vis = [n for n in range(N) if (not causal) or (m + N - M >= n)]
                if not vis:
                    continue
                s = []
                for n in vis:
                    far = m + N - M - n >= w
                    s.append(sm_scale * float(np.dot(q2[b, h, m], k2[b, h, n]) if far else np.dot(q1[b, h, m], k1[b, h, n])))
                top = max(s)
                e = [math.exp(x - top) for x in s]
                z = sum(e)
                for n, en in zip(vis, e):
                    o[b, h, m] += (en / z) * v[b, h, n]
    return o


def paged(q, kc, vc, lens, table, scale):
    """q (S, Hq, D); caches (blocks, Hkv, block, D); token t of sequence s sits in cache block
    table[s, t // block] at slot t % block; query head h uses kv head h // (Hq / Hkv)."""
    S, Hq, D = q.shape
    Hkv, bs = kc.shape[1], kc.shape[2]
    out = np.zeros((S, Hq, D))
    for s in range(S):
        for h in range(Hq):
            hk = h // (Hq // Hkv)
            sc = [scale * float(np.dot(q[s, h], kc[table[s, t // bs], hk, t % bs])) for t in range(lens[s])]
            top = max(sc)
            e = [math.exp(x - top) for x in sc]
            z = sum(e)
            for t, et in enumerate(e):
                out[s, h] += (et / z) * vc[table[s, t // bs], hk, t % bs]
    return out


def main():
    rng = np.random.default_rng(20240607)
    data = {}
    # flash: (name, B, H, Hk, M, N, D, causal)
    for name, B, H, Hk, M, N, D, causal in [("flash_causal_gqa", 1, 4, 2, 37, 50, 32, True),
                                            ("flash_rows_without_keys", 1, 2, 2, 40, 9, 16, True),
                                            ("flash_noncausal", 2, 2, 1, 21, 33, 64, False)]:
        q, k, v = f16(rng, (B, H, M, D)), f16(rng, (B, Hk, N, D)), f16(rng, (B, Hk, N, D))
        sm = 1.0 / math.sqrt(D)
        o, L, tot = flash(q, k, v, causal, sm)
        data.update({f"{name}.q": q, f"{name}.k": k, f"{name}.v": v, f"{name}.causal": np.array(causal),
                     f"{name}.o": o, f"{name}.L": L, f"{name}.tot": tot})
    for name, B, H, M, N, D, w, causal in [("piecewise_causal", 1, 2, 45, 45, 32, 11, True),
                                           ("piecewise_noncausal_cross", 1, 1, 20, 41, 16, -5, False)]:
        q1, q2 = f16(rng, (B, H, M, D)), f16(rng, (B, H, M, D))
        k1, k2, v = f16(rng, (B, H, N, D)), f16(rng, (B, H, N, D)), f16(rng, (B, H, N, D))
        o = piecewise(q1, k1, q2, k2, v, w, causal, 1.0 / math.sqrt(D))
        data.update({f"{name}.q1": q1, f"{name}.k1": k1, f"{name}.q2": q2, f"{name}.k2": k2, f"{name}.v": v,
                     f"{name}.w": np.array(w), f"{name}.causal": np.array(causal), f"{name}.o": o})
    S, Hq, Hkv, D, bs, nb = 3, 4, 2, 32, 16, 12
    lens = np.array([40, 1, 17], dtype=np.int32)
    q = f16(rng, (S, Hq, D), D ** -0.5)
    kc, vc = f16(rng, (nb, Hkv, bs, D), D ** -0.5), f16(rng, (nb, Hkv, bs, D), D ** -0.5)
    table = rng.permutation(nb)[:9].reshape(S, 3).astype(np.int64)
    data.update({"paged.q": q, "paged.kc": kc, "paged.vc": vc, "paged.lens": lens, "paged.table": table,
                 "paged.out": paged(q, kc, vc, lens, table, D ** -0.5)})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_vectors.npz")
    # inputs are exact in fp16; expected outputs are kept in fp32
    packed = {}
    for key, val in data.items():
        is_expected = key.split(".")[1] in ("o", "L", "tot", "out")
        packed[key] = val.astype(np.float32) if is_expected else (val.astype(np.float16) if val.dtype == np.float64 else val)
    np.savez_compressed(path, **packed)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
