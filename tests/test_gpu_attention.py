"""RoPE + KV-cache store and causal attention kernels against the oracle's literal
MultiHeadSelfAttention pieces (split heads, RoPE, per-head q.k^T*scale + mask, softmax, p.v,
merge) on the same inputs: prefill chunks, then single-row decode steps over the growing
cache (split-K path), for head dims 32/64/128."""
import numpy as np
import pytest

from deepj_amd.fused import (DeviceBuffers, Stream, attention_scratch_floats, attn_decode_scratch_floats,
                             attn_record_floats)
from oracle import cpu_ref as ref
from gpu_util import assert_close

pytestmark = pytest.mark.gpu


def gaussian(rows, cols, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal((rows, cols)) * scale).astype(np.float32)


def oracle_attention(q, k, v, H, cos, sin):
    """merged attention output for all rows, literal reference path."""
    qh = ref.rope_apply(ref.split_heads(q, H), q.shape[0], H, cos, sin)
    kh = ref.rope_apply(ref.split_heads(k, H), q.shape[0], H, cos, sin)
    vh = ref.split_heads(v, H)
    return ref.merge_heads(ref.attention_heads(qh, kh, vh, H, causal=True), H)


@pytest.mark.parametrize("H,hd,max_seq,chunks", [(8, 32, 256, [32, 1, 1, 1]), (4, 64, 200, [70, 1, 1, 60, 1]),
                                                 (2, 128, 130, [5, 1, 124]), (32, 64, 2048, [3, 1]),
                                                 # grids of 288 and 576 workgroups at 128 rows each: the prefill kernel's
                                                 # two-key-set and one-key-set variants (the small shapes above use four)
                                                 (32, 64, 1200, [1100, 1, 20]), (64, 32, 1150, [1100, 1]),
                                                 # the value products on bf16 planes: one key set at 64-wide heads, two at
                                                 # 128-wide ones (narrower heads with two or four sets keep the fp32 form)
                                                 (64, 64, 1100, [1050, 1, 17]), (32, 128, 1150, [1100, 3]),
                                                 # ragged chunks around the 16-row threshold and the 32-row query tile
                                                 (4, 64, 200, [17, 1, 33, 15, 16, 65]), (3, 128, 150, [31, 97]),
                                                 # short continuations of a cached prefix (2 to 32 rows: the key rounds
                                                 # of a head are dealt to several workgroups whose records a second
                                                 # kernel merges), ragged, after prefixes of less than one round of
                                                 # keys and of many; with few heads (eight shares) and with 256 (one)
                                                 (32, 64, 2048, [515, 2, 7, 15, 8, 32, 1, 31, 900, 5]), (4, 128, 700, [600, 7, 2, 8, 15]),
                                                 (8, 32, 300, [2, 3, 31, 7, 130, 9]), (256, 32, 40, [20, 3, 8, 4, 5])])
def test_rope_store_attention_prefill_and_decode(H, hd, max_seq, chunks):
    d = H * hd
    total = sum(chunks)
    layers, layer = 2, 1                                 # exercise the per-layer offset
    q, k, v = (gaussian(total, d, 10 + i) for i in range(3))
    cos, sin = ref.rope_tables(hd, max_seq)
    exp = oracle_attention(q, k, v, H, cos, sin)

    dev = DeviceBuffers()
    try:
        kc, vc = dev.alloc(layers * max_seq * d), dev.alloc(layers * max_seq * d)
        state = dev.upload(np.zeros(4, np.int32))
        cos_b, sin_b = dev.upload(cos), dev.upload(sin)
        sf = attention_scratch_floats(H, hd, max_seq)
        scratch = dev.alloc(sf)
        tok, tokens = dev.upload(np.zeros(4, np.int32)), dev.alloc(max_seq)
        Stream().fill(scratch, 0, sf).run()
        pos = 0
        for S in chunks:
            qkv = np.concatenate([q[pos:pos + S], k[pos:pos + S], v[pos:pos + S]], axis=1)
            qkv_b, q_b, out_b = dev.upload(qkv), dev.alloc(S * d), dev.alloc(S * d)
            (Stream().rope_kv_store(qkv_b, q_b, kc, vc, state, cos_b, sin_b, S, H, hd, max_seq, layer)
             .attention(q_b, kc, vc, out_b, state, scratch, S, H, hd, max_seq, layer)
             .decode_advance(state, tok, tokens, max_seq, S).run())
            got = dev.download(out_b, (S, d))
            assert_close(exp[pos:pos + S], got, atol=2e-5, rtol=1e-4, what=f"rows {pos}..{pos + S} of {chunks}")
            dev.release(qkv_b, q_b, out_b)
            pos += S
        st = dev.download(state, (4,), np.int32)
        assert st[0] == total and st[2] == len(chunks)
    finally:
        dev.release_all()


@pytest.mark.parametrize("H,hd,max_seq,prefill,steps", [(8, 32, 256, 32, 5), (32, 64, 2048, 515, 3), (4, 128, 96, 1, 40)])
def test_fused_decode_attention_and_decode_next(H, hd, max_seq, prefill, steps):
    """ATTN_DECODE (rotate + append + split attention + merge) over a growing cache, then
    DECODE_NEXT (argmax, advance, embedding gather) - the two fused ops of a decode step."""
    d = H * hd
    total = prefill + steps
    q, k, v = (gaussian(total, d, 30 + i) for i in range(3))
    cos, sin = ref.rope_tables(hd, max_seq)
    exp = oracle_attention(q, k, v, H, cos, sin)
    dev = DeviceBuffers()
    try:
        kc, vc = dev.alloc(max_seq * d), dev.alloc(max_seq * d)
        state = dev.upload(np.zeros(4, np.int32))
        cos_b, sin_b = dev.upload(cos), dev.upload(sin)
        sf = attention_scratch_floats(H, hd, max_seq)
        scratch, scratch_dec = dev.alloc(sf), dev.alloc(attn_decode_scratch_floats(H, hd))
        Stream().fill(scratch, 0, sf).run()
        tok, tokens = dev.upload(np.zeros(4, np.int32)), dev.alloc(max_seq)
        qkv0 = np.concatenate([q[:prefill], k[:prefill], v[:prefill]], axis=1)
        qkv_b, q_b, out_b = dev.upload(qkv0), dev.alloc(prefill * d), dev.alloc(prefill * d)
        (Stream().rope_kv_store(qkv_b, q_b, kc, vc, state, cos_b, sin_b, prefill, H, hd, max_seq, 0)
         .attention(q_b, kc, vc, out_b, state, scratch, prefill, H, hd, max_seq, 0)
         .decode_advance(state, tok, tokens, max_seq, prefill).run())
        assert_close(exp[:prefill], dev.download(out_b, (prefill, d)), atol=2e-5, rtol=1e-4)
        vocab = 50
        table = gaussian(vocab, d, 40)
        logits_b, x_b, row_b, o_b = dev.alloc(vocab), dev.alloc(d), dev.alloc(3 * d), dev.alloc(d)
        for i in range(steps):
            p = prefill + i
            dev.write(row_b, np.concatenate([q[p], k[p], v[p]]))
            logits = gaussian(1, vocab, 50 + i)
            dev.write(logits_b, logits)
            (Stream().attn_decode(row_b, kc, vc, o_b, state, scratch_dec, cos_b, sin_b, H, hd, max_seq, 0)
             .decode_next(logits_b, state, tokens, max_seq, dev.upload(table), x_b, vocab, d).run())
            assert_close(exp[p:p + 1], dev.download(o_b, (1, d)), atol=2e-5, rtol=1e-4, what=f"decode step {i}")
            st = dev.download(state, (4,), np.int32)
            best = int(np.argmax(logits))
            assert (st[0], st[1], st[2]) == (p + 1, best, 2 + i)
            assert np.array_equal(dev.download(x_b, (d,)), table[best])
        # the appended rows really are in the cache: a plain ATTENTION over the cache agrees
        st = np.array([total - 1, 0, 0, 0], np.int32); dev.write(state, st)
        qr = ref.merge_heads(ref.rope_apply(ref.split_heads(q, H), total, H, cos, sin), H)[total - 1:]
        (Stream().attention(dev.upload(qr), kc, vc, o_b, state, scratch, 1, H, hd, max_seq, 0).run())
        assert_close(exp[total - 1:], dev.download(o_b, (1, d)), atol=2e-5, rtol=1e-4)
    finally:
        dev.release_all()


@pytest.mark.parametrize("vocab", [50, 4099, 32000, 40001])
def test_decode_next_orders_logits_like_float_compare(vocab):
    """DECODE_NEXT picks what TextGenerator's stable descending sort puts first (TextGenerator.java:163-170 with
    Float.compare): the largest value, the lowest index among equals, NaN above everything (the first NaN wins),
    index 0 when every logit is -inf; vocabularies below, at and beyond one round of the kernel's loads and not a
    multiple of four."""
    d = 8
    rng = np.random.default_rng(vocab)
    table = gaussian(vocab, d, 7)
    cases = []
    base = (rng.standard_normal(vocab) * 3).astype(np.float32)
    cases.append((base.copy(), int(np.argmax(base))))
    t = base.copy(); hi = float(t.max()) + 1.0
    for i in (vocab - 1, vocab // 2, 3): t[i] = hi
    cases.append((t, 3))                                            # ties: lowest index
    t = base.copy(); t[vocab - 2] = np.nan; t[vocab // 3] = np.nan; t[1] = np.inf
    cases.append((t, vocab // 3))                                   # NaN outranks +inf; the first NaN wins
    cases.append((np.full(vocab, -np.inf, np.float32), 0))          # nothing is larger than anything: index 0
    t = np.full(vocab, -np.inf, np.float32); t[vocab - 1] = -1e30
    cases.append((t, vocab - 1))
    dev = DeviceBuffers()
    try:
        state, tokens = dev.upload(np.zeros(4, np.int32)), dev.alloc(64)
        logits_b, x_b, table_b = dev.alloc(vocab), dev.alloc(d), dev.upload(table)
        for n, (logits, want) in enumerate(cases):
            dev.write(logits_b, logits)
            Stream().decode_next(logits_b, state, tokens, 64, table_b, x_b, vocab, d).run()
            st = dev.download(state, (4,), np.int32)
            assert (st[0], st[1], st[2]) == (n + 1, want, n + 1), f"case {n}: {st}"
            assert np.array_equal(dev.download(x_b, (d,)), table[want])
        got = dev.download(tokens, (64,), np.int32)[:len(cases)]
        assert list(got) == [w for _, w in cases]
    finally:
        dev.release_all()


@pytest.mark.parametrize("H,hd,max_seq,start,steps", [(8, 32, 256, 0, 6), (32, 64, 2048, 515, 3), (4, 128, 96, 55, 41),
                                                      (2, 64, 1, 0, 1), (5, 32, 700, 509, 5),
                                                      # splits longer than one key/value round (two rounds in flight),
                                                      # and longer than two (the loop comes round again)
                                                      (32, 64, 2048, 1500, 2), (4, 128, 700, 600, 3), (2, 128, 1100, 1090, 3)])
def test_decode_attention_records_merged_by_the_q8_linear_prologue(H, hd, max_seq, start, steps):
    """ATTN_DECODE_RECORDS leaves one record per (head, key split); the ATTN_MERGE prologue of the following
    Q8_LINEAR merges them.  With an identity-like projection out of reach (Q8), the check is against the oracle's
    attention row pushed through the dequantised weight, plus a residual; positions from an empty cache (three
    of the four splits have no key) to the last row of the cache."""
    from deepj_amd import HipNative
    d = H * hd
    total = start + steps
    q, k, v = (gaussian(total, d, 60 + i) for i in range(3))
    cos, sin = ref.rope_tables(hd, max_seq)
    exp_att = oracle_attention(q, k, v, H, cos, sin)
    n_out = 48
    w = gaussian(d, n_out, 70, 0.05)
    res = gaussian(1, n_out, 71)
    wdq = ref.q8_roundtrip(w)
    dev = DeviceBuffers()
    try:
        kc, vc = dev.alloc(max_seq * d), dev.alloc(max_seq * d)
        state = dev.upload(np.zeros(4, np.int32))
        cos_b, sin_b = dev.upload(cos), dev.upload(sin)
        if start:
            sf = attention_scratch_floats(H, hd, max_seq)
            scratch = dev.alloc(sf)
            qkv0 = np.concatenate([q[:start], k[:start], v[:start]], axis=1)
            qkv_b, q_b = dev.upload(qkv0), dev.alloc(start * d)
            Stream().rope_kv_store(qkv_b, q_b, kc, vc, state, cos_b, sin_b, start, H, hd, max_seq, 0).run()
        wsrc, wq = dev.upload(w), dev.alloc(HipNative.q8Floats(d, n_out))
        Stream().q8_quantize(wsrc, wq, d, n_out).run()
        rec = dev.alloc(attn_record_floats(H, hd))
        row_b, out_b, res_b, att_b = dev.alloc(3 * d), dev.alloc(n_out), dev.upload(res), dev.alloc(d)
        scratch_dec = dev.alloc(attn_decode_scratch_floats(H, hd))
        for i in range(steps):
            p = start + i
            dev.write(state, np.array([p, 0, 0, 0], np.int32))
            dev.write(row_b, np.concatenate([q[p], k[p], v[p]]))
            (Stream().attn_decode_records(row_b, kc, vc, rec, state, cos_b, sin_b, H, hd, max_seq, 0)
             .q8_linear(rec, wq, out_b, 1, d, n_out, residual=res_b, attn_merge_hd=hd).run())
            exp = ref.add(res, ref.matmul(exp_att[p:p + 1], wdq))
            scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
            assert_close(exp, dev.download(out_b, (1, n_out)), atol=1e-4 * scale, rtol=1e-4, what=f"step {i} at position {p}")
            # the merging path and the self-merging ATTN_DECODE agree on the attention row itself (the row was
            # appended by the first of them; the second rewrites the same values)
            Stream().attn_decode(row_b, kc, vc, att_b, state, scratch_dec, cos_b, sin_b, H, hd, max_seq, 0).run()
            assert_close(exp_att[p:p + 1], dev.download(att_b, (1, d)), atol=2e-5, rtol=1e-4, what=f"row {p}")
    finally:
        dev.release_all()


def test_attn_merge_prologue_rejects_bad_combinations():
    from deepj_amd import opcodes as op
    dev = DeviceBuffers()
    try:
        rec, w, out, g = dev.alloc(attn_record_floats(2, 32)), dev.alloc(4096), dev.alloc(64), dev.alloc(64)
        for flags, m, hd in ((op.LIN_ATTN_MERGE | op.LIN_RMSNORM, 1, 32), (op.LIN_ATTN_MERGE | op.LIN_GELU, 1, 32),
                             (op.LIN_ATTN_MERGE, 2, 32), (op.LIN_ATTN_MERGE, 1, 48), (op.LIN_ATTN_MERGE, 1, 128)):
            with pytest.raises(RuntimeError, match="OP_Q8_LINEAR"):
                Stream().emit(op.OP_Q8_LINEAR, rec, w, out, m, 64, 4, flags, hd, -1, -1, -1).run()
        small = dev.alloc(8)
        with pytest.raises(RuntimeError, match="op needs"):
            Stream().emit(op.OP_Q8_LINEAR, small, w, out, 1, 64, 4, op.LIN_ATTN_MERGE, 32, -1, -1, -1).run()
        del g
    finally:
        dev.release_all()


def test_rope_rows_and_attention_over_token_major_kv():
    H, hd, max_seq, n = 4, 32, 64, 37
    d = H * hd
    q, k, v = (gaussian(n, d, 20 + i) for i in range(3))
    cos, sin = ref.rope_tables(hd, max_seq)
    exp = oracle_attention(q, k, v, H, cos, sin)
    dev = DeviceBuffers()
    try:
        state = dev.upload(np.array([n - 1, 0, 0, 0], np.int32))      # the query is the last row
        cos_b, sin_b = dev.upload(cos), dev.upload(sin)
        kpad = np.zeros((max_seq, d), np.float32); kpad[:n] = k
        vpad = np.zeros((max_seq, d), np.float32); vpad[:n] = v
        k_b, kr_b, v_b = dev.upload(kpad), dev.alloc(max_seq * d), dev.upload(vpad)
        q_b, qr_b, out_b = dev.upload(q[n - 1:]), dev.alloc(d), dev.alloc(d)
        sf = attention_scratch_floats(H, hd, max_seq)
        scratch = dev.alloc(sf)
        (Stream().fill(scratch, 0, sf)
         .rope_rows(k_b, kr_b, state, cos_b, sin_b, max_seq, H, hd, max_seq, True)      # position = row
         .rope_rows(q_b, qr_b, state, cos_b, sin_b, 1, H, hd, max_seq, False)           # position = state[0]
         .attention_kv(qr_b, kr_b, v_b, out_b, state, scratch, 1, H, hd, max_seq).run())
        assert_close(exp[n - 1:], dev.download(out_b, (1, d)), atol=2e-5, rtol=1e-4)
        kr = dev.download(kr_b, (max_seq, d))
        assert_close(ref.merge_heads(ref.rope_apply(ref.split_heads(k, H), n, H, cos, sin), H), kr[:n], 1e-6, 1e-6)
    finally:
        dev.release_all()


def test_attention_rejects_bad_shapes():
    dev = DeviceBuffers()
    try:
        b = dev.alloc(64)
        with pytest.raises(RuntimeError, match="head dim must be 32, 64 or 128"):
            Stream().attention(b, b, b, b, b, b, 1, 1, 48, 1, 0).run()
        with pytest.raises(RuntimeError, match="op needs"):
            Stream().attention(b, b, b, b, b, b, 1, 2, 32, 64, 0).run()       # cache too small
    finally:
        dev.release_all()
