#!/usr/bin/env python3
"""Adds "fp64_step0" to the entries of tests/golden/model_greedy.json: a float64 evaluation (numpy) of the prompt
forward of each full-size configuration, next to the CPU oracle's fp32 value and to a second fp32 evaluation in a
different summation order (numpy's blocked single-precision products).

Why: at full size the reference's own fp32 arithmetic (sequential fp32 sums over 768..11008 terms, 8-16 layers
deep, random-init weights that make logits of +-20) sits some 1e-3 (max-abs) away from the exact result, so no
implementation with a different summation order can be asked to agree with it to 1e-3.  The fixture stores, for a
set of logit columns of the last prompt row, the float64 value (same Q8-dequantised weights, same formulas, the
model's fp32 constants) and the oracle's fp32 value, so the GPU test can check that the GPU result is as close to
exact arithmetic as the CPU path is; the second fp32 order shows how far two correct fp32 evaluations of the same
model are apart (for the DeepSeek model at the reference's initialisation: by O(1)).

    python tests/golden/make_fp64_probe.py c3 [c4] [c5] [c5_ref_init] [g2]     # minutes per configuration on 8 cores
"""
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import cpu_ref as ref  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "model_greedy.json")


def forward_last_row(m, prompt, f):
    """Logits of the last prompt row in dtype f (float64: the exact reference value up to 1e-13; float32: the same
    model in numpy's summation order).  Formulas as the oracle's model_ref.c / the reference's layers."""
    S, D, H, L, V = len(prompt), m.d, m.heads, m.layers, m.vocab
    hd = D // H
    kind = m.kind
    w = lambda n: m.weight(n).astype(f)  # noqa: E731
    scale = f(np.float32(1.0 / np.sqrt(hd)))            # MultiHeadSelfAttention.java:45
    mask = np.triu(np.full((S, S), f(np.float32(-1e9))), 1)

    def rmsnorm(x, g):                                  # RMSNorm1D.java:46-57, eps 1e-6f
        return g * x / np.sqrt((x * x).mean(1, keepdims=True) + f(np.float32(1e-6)))

    def layernorm(x, g, b):                             # LayerNorm1D.java:34-66, eps 1e-5f, population variance
        mu = x.mean(1, keepdims=True)
        var = ((x - mu) ** 2).mean(1, keepdims=True)
        return (x - mu) / np.sqrt(var + f(np.float32(1e-5))) * g + b

    rotate = kind != 2
    if rotate:
        cos, sin = ref.rope_tables(hd, m.max_seq)
        cos, sin = cos[:S].astype(f), sin[:S].astype(f)

    def rope(t):                                        # RotaryEmbedding.java:112-122, pairs (2i, 2i+1)
        t = t.reshape(S, H, hd // 2, 2)
        if not rotate:
            return t.reshape(S, H, hd)
        o = np.empty_like(t)
        o[..., 0] = t[..., 0] * cos[:, None, :] - t[..., 1] * sin[:, None, :]
        o[..., 1] = t[..., 0] * sin[:, None, :] + t[..., 1] * cos[:, None, :]
        return o.reshape(S, H, hd)

    def attention(q, k, v):                             # HeadOps.java:90-140
        q, k, v = rope(q), rope(k), v.reshape(S, H, hd)
        out = np.empty((S, H, hd), dtype=f)
        for h in range(H):
            s = q[:, h] @ k[:, h].T * scale + mask
            p = np.exp(s - s.max(1, keepdims=True))
            p /= p.sum(1, keepdims=True)
            out[:, h] = p @ v[:, h]
        return out.reshape(S, D)

    x = w("emb")[prompt]
    if kind == 2:
        x = x + w("pos")[:S]                            # GPTModel.java:52-54
    for l in range(L):
        P = f"L{l}."
        if kind == 2:                                   # GPTTransformerBlock.java:65-73
            h = layernorm(x, w(P + "g1"), w(P + "be1"))
            x2 = x + attention(h @ w(P + "wq"), h @ w(P + "wk"), h @ w(P + "wv")) @ w(P + "wo")
            h = layernorm(x2, w(P + "g2"), w(P + "be2"))
            z = h @ w(P + "wg") + w(P + "bg")
            c = f(np.sqrt(np.float32(2.0) / np.float32(np.pi)))               # CpuBackend.java:338
            z = f(0.5) * z * (1 + np.tanh(c * (z + f(np.float32(0.044715)) * z * z * z)))
            x = x2 + z @ w(P + "wd") + w(P + "bd")
            continue
        h = rmsnorm(x, w(P + "g1"))
        if kind == 1:                                   # MultiHeadLatentAttention.java:92-123
            cq, ckv = h @ w(P + "wdq"), h @ w(P + "wdkv")
            att = attention(cq @ w(P + "wuq"), ckv @ w(P + "wuk"), ckv @ w(P + "wuv"))
        else:                                           # MultiHeadSelfAttention.java:60-86
            att = attention(h @ w(P + "wq"), h @ w(P + "wk"), h @ w(P + "wv"))
        x2 = x + att @ w(P + "wo")
        h = rmsnorm(x2, w(P + "g2"))                    # SwiGLULayer.java:63-70
        g = h @ w(P + "wg") + w(P + "bg")
        u = h @ w(P + "wu") + w(P + "bu")
        x = x2 + ((g / (1 + np.exp(-g))) * u) @ w(P + "wd") + w(P + "bd")
    last = x[-1:]
    last = layernorm(last, w("gf"), w("bf")) if kind == 2 else rmsnorm(last, w("gf"))
    return (last @ w("wlm") + w("blm"))[0]


def build_oracle(c):
    m = ref.Model(seed=c["seed"], **c["model"])
    if "mla_weight_scale" in c:
        for n in m.weight_names():
            if n.split(".")[-1] in ("wdq", "wuq", "wdkv", "wuk", "wuv"):
                m.weight(n)[...] *= np.float32(c["mla_weight_scale"])
    m.q8_roundtrip()
    return m


def run(name, data):
    c = data[name]["config"]
    ref.set_threads(os.cpu_count() or 1)
    ref.set_column_parallel(True)
    t0 = time.time()
    m = build_oracle(c)
    V = c["model"]["vocab"]
    prompt = ref.JavaRandom(c["prompt_seed"]).ints(c["prompt_len"], V)
    m.reset_cache()
    oracle = m.forward_cached(prompt, last_only=True)[0].astype(np.float64)
    print(f"[{name}] oracle prompt forward {time.time() - t0:.0f}s", flush=True)
    t0 = time.time()
    exact = forward_last_row(m, prompt, np.float64)
    alt = forward_last_row(m, prompt, np.float32).astype(np.float64)
    print(f"[{name}] float64 and second fp32 evaluation {time.time() - t0:.0f}s", flush=True)
    cols = sorted(set(list(range(0, V, 250)) + [int(np.argmax(exact)), int(np.argmin(exact))]))
    srt = np.sort(exact)
    data[name]["fp64_step0"] = {
        "cols": cols,
        "fp64": [float(exact[j]) for j in cols],
        "oracle_fp32": [float(oracle[j]) for j in cols],
        "oracle_max_abs_err_all_cols": float(np.max(np.abs(oracle - exact))),
        "oracle_rms_err_all_cols": float(np.sqrt(np.mean((oracle - exact) ** 2))),
        "alt_fp32_max_abs_err_all_cols": float(np.max(np.abs(alt - exact))),
        "alt_fp32_rms_err_all_cols": float(np.sqrt(np.mean((alt - exact) ** 2))),
        "alt_fp32_vs_oracle_max_abs": float(np.max(np.abs(alt - oracle))),
        "fp64_top2_gap": float(srt[-1] - srt[-2]),
        "fp64_argmax": int(np.argmax(exact)),
    }
    f = data[name]["fp64_step0"]
    print(f"[{name}] vs float64: oracle max-abs {f['oracle_max_abs_err_all_cols']:.3e} rms {f['oracle_rms_err_all_cols']:.3e}; "
          f"second fp32 order max-abs {f['alt_fp32_max_abs_err_all_cols']:.3e}; the two fp32 orders apart by "
          f"{f['alt_fp32_vs_oracle_max_abs']:.3e}", flush=True)
    m.close()


if __name__ == "__main__":
    names = sys.argv[1:] or ["c3"]
    data = json.load(open(OUT))
    for n in names:
        run(n, data)
        json.dump(data, open(OUT, "w"), indent=1)
