"""The many-row Q8 GEMM on fp16 matrix cores (two-piece activations, direct loads into LDS) through the C ABI against
the CPU oracle: fp32 CpuBackend.matmul (tensor/cpu/CpuBackend.java:168-188, ikj order) on the dequantised weights.

Shapes are chosen so that the library takes this kernel (HipNative.q8GemmPath says so for each), with its 128-row
and its 64-row workgroup tile (the shapes with about 160 tiles or more of 128 x 256 take the former); what the tests vary:
ragged M and N (not multiples of the 128 x 256 tile), K that is not a multiple of the 32-group, every epilogue
(bias, GELU, residual, interleaved SwiGLU with both biases), the RMSNorm / LayerNorm prologue, rows whose magnitudes span
twelve decades with outliers and tiny values inside a row, all-zero rows, K shared by several workgroups whose partial
products a second kernel sums (few tiles, long K), prepared weights (OP_Q8_PREPARE) against
per-call conversion, and the loss of that association when the weights are rewritten.
Gate: |expected - actual| <= atol + 1e-4 |expected| with atol = 1e-4 of the output's rms (the per-op gate of
src/test/java/io/github/kirstenali/deepj/tensor/metal/MetalBackendTest.java:452-466)."""
import numpy as np
import pytest

from deepj_amd import HipNative, JavaRandom
from deepj_amd.fused import DeviceBuffers, Stream
from oracle import cpu_ref as ref
from gpu_util import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    ref.set_threads(ref.default_threads())
    d = DeviceBuffers()
    yield d
    d.release_all()
    ref.set_threads(1)


def quantised(dev, w):
    """Uploads w [K x N], quantises it with the library and returns (buffer, the oracle's dequantised copy)."""
    k, n = w.shape
    src = dev.upload(w)
    wq = dev.alloc(HipNative.q8Floats(k, n))
    Stream().q8_quantize(src, wq, k, n).run()
    dev.release(src)
    return wq, ref.q8_roundtrip(w)


def gate(exp):
    return 1e-4 * float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))


def test_path_query_matches_the_documented_rule():
    assert HipNative.q8GemmPath(512, 2048, 11264) == 128      # 4 x 59 tiles of 128 x 192 (4 x 44 of 128 x 256 leave 80 compute units idle)
    assert HipNative.q8GemmPath(2048, 4096, 4096) == 128      # 16 x 16
    assert HipNative.q8GemmPath(512, 2048, 6144) == 64        # 96 such tiles would idle most of the chip: 192 of 64 x 256
    assert HipNative.q8GemmPath(512, 2048, 2048) == 64        # 64 even of those: four workgroups share each tile's K
    assert HipNative.q8GemmPath(512, 1024, 2048) == 0         # ... when K is 1536 or more: else the bf16 kernels
    assert HipNative.q8GemmTile(256, 2048, 6144) == (64, 192, 2)     # 128 narrow tiles, two shares each: every compute unit
    assert HipNative.q8GemmTile(320, 2048, 2048) == (64, 256, 6)     # shares of at least eight K steps
    assert HipNative.q8GemmTile(256, 2048, 2048) == (0, 0, 1)        # too little to stream for eight shares' partial products
    assert HipNative.q8GemmTile(128, 2048, 11264) == (0, 0, 1)       # fewer than 256 rows: not without prepared weights
    assert HipNative.q8GemmTilePrepared(128, 2048, 11264) == (64, 192, 2)
    assert HipNative.q8GemmTilePrepared(15, 2048, 11264) == (0, 0, 1)
    assert HipNative.q8GemmTilePrepared(64, 2048, 2048) == (0, 0, 1)
    assert HipNative.q8GemmPath(512, 5632, 2048) == 64        # the same 64 tiles over a long K: four workgroups share each
    assert HipNative.q8GemmTile(512, 5632, 2048) == (64, 256, 4)
    assert HipNative.q8GemmTile(512, 2048, 6144) == (64, 192, 1)     # 256 tiles: one per compute unit
    assert HipNative.q8GemmTile(512, 2048, 11264) == (128, 192, 1)
    assert HipNative.q8GemmTile(2048, 4096, 12288) == (128, 256, 1)  # several rounds of tiles: the large one
    assert HipNative.q8GemmTile(8, 2048, 2048) == (0, 0, 1)
    assert HipNative.q8GemmPath(1, 2048, 32000) == 0          # the matvec's case
    assert HipNative.q8GemmPath(512, 2048, 11266) == 0        # four columns per lane in the epilogue
    # fp16 rows padded to a multiple of 768 (both tile widths), the transposed scales, 64 floats of slack
    assert HipNative.q8PreparedFloats(2048, 11264) == (11520 * (2048 + 64)) // 2 + 64 * 11520 + 64


@pytest.mark.parametrize("m,k,n,tile", [(300, 1000, 13828, 128), (257, 96, 40964, 128), (640, 2048, 8192, 128),
                                         (300, 1000, 8196, 64), (512, 2048, 6144, 64), (257, 96, 13000, 64)])
def test_plain_product_ragged_shapes(dev, m, k, n, tile):
    assert HipNative.q8GemmPath(m, k, n) == tile
    w = JavaRandom(11).tensor(k, n, 0.02)
    x = JavaRandom(12).tensor(m, k, 1.0)
    wq, deq = quantised(dev, w)
    exp = ref.matmul(x, deq)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    Stream().q8_linear(xb, wq, ob, m, k, n).run()
    got = dev.download(ob, (m, n))
    dev.release(xb, ob, wq)
    assert_close(exp, got, atol=gate(exp), rtol=1e-4, what=f"Q8 linear M={m} K={k} N={n}")


@pytest.mark.parametrize("m,k,n,shares", [(256, 4096, 2048, 8), (512, 2048, 2048, 4), (384, 4096, 2048, 5), (320, 2048, 4096, 3),
                                           (300, 4096, 2044, 6)])
def test_every_way_the_shares_of_k_are_dealt_to_the_xcds(dev, m, k, n, shares):
    """A tile's K shares go to workgroups by one of two rules: share counts that divide eight put one share on each XCD
    (eight and four here), the others keep every share of a column tile together (six, five and three).  Each must cover every
    (row tile, column tile, share) exactly once: a tile missed or taken twice shows as a wrong block of the product."""
    assert HipNative.q8GemmTile(m, k, n) == (64, 256, shares)
    w = JavaRandom(41).tensor(k, n, 0.02)
    x = JavaRandom(42).tensor(m, k, 1.0)
    b = JavaRandom(43).tensor(1, n, 0.3)
    wq, deq = quantised(dev, w)
    exp = ref.add_row_vector(ref.matmul(x, deq), b)
    xb, bb, ob = dev.upload(x), dev.upload(b), dev.alloc(m * n)
    Stream().q8_linear(xb, wq, ob, m, k, n, bias=bb).run()
    got = dev.download(ob, (m, n))
    dev.release(xb, bb, ob, wq)
    assert_close(exp, got, atol=gate(exp), rtol=1e-4, what=f"Q8 linear M={m} K={k} N={n}, K shared by {shares}")


@pytest.mark.parametrize("m,k,n,tile,epilogue", [
    (64, 4096, 11008, (64, 192, 4), "bias"),              # a short prompt against a wide projection: four shares of K
    (16, 2048, 5632, (64, 192, 4), "swiglu"),             # the fewest rows taken; three quarters of a tile's rows are padding
    (100, 2048, 6144, (64, 192, 4), "rms_bias"),          # ragged rows, the RMSNorm prologue
    (200, 1000, 11268, (64, 192, 1), "residual"),         # ragged everything, K not shared
    (255, 5632, 2048, (64, 256, 8), "bias_residual"),     # a narrow output that qualifies through its long K: eight shares
])
def test_fewer_than_256_rows_on_prepared_weights(dev, m, k, n, tile, epilogue):
    """With the weights already in the fp16 GEMM's layout the library takes prompts from 16 rows on, where its plan
    expects enough workgroups (deepj_hip_q8_gemm_tile_prepared); without them the same shapes stay on the bf16 kernels.
    Both against the oracle."""
    swiglu = epilogue == "swiglu"
    n_rows = 2 * n if swiglu else n
    assert HipNative.q8GemmTile(m, k, n_rows) == (0, 0, 1)
    assert HipNative.q8GemmTilePrepared(m, k, n_rows) == tile
    x = JavaRandom(51).tensor(m, k, 1.0)
    b = JavaRandom(53).tensor(1, n, 0.3)
    r = JavaRandom(54).tensor(m, n, 1.0)
    g = (1.0 + 0.1 * JavaRandom(55).tensor(1, k, 1.0)).astype(np.float32)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    kw = {}
    if swiglu:
        wg, wu = JavaRandom(52).tensor(k, n, 0.03), JavaRandom(56).tensor(k, n, 0.03)
        inter = np.empty((k, 2 * n), np.float32)
        inter[:, 0::2], inter[:, 1::2] = wg, wu
        wq, deq = quantised(dev, inter)
        exp = ref.multiply(ref.silu(ref.matmul(x, np.ascontiguousarray(deq[:, 0::2]))), ref.matmul(x, np.ascontiguousarray(deq[:, 1::2])))
        kw["swiglu"] = True
    else:
        wq, deq = quantised(dev, JavaRandom(52).tensor(k, n, 0.03))
        xin = x
        if epilogue.startswith("rms"):
            xin = ref.rmsnorm(x, g)
            kw["gamma"] = dev.upload(g)
        exp = ref.matmul(xin, deq)
        if "bias" in epilogue:
            exp = ref.add_row_vector(exp, b)
            kw["bias"] = dev.upload(b)
        if "residual" in epilogue:
            exp = ref.add(r, exp)
            kw["residual"] = dev.upload(r)
    op = Stream().q8_linear(xb, wq, ob, m, k, n, **kw)
    op.run()
    unprepared = dev.download(ob, (m, n))
    assert_close(exp, unprepared, atol=gate(exp), rtol=1e-4, what=f"bf16 kernels M={m} K={k} N={n} {epilogue}")
    prep = dev.alloc(HipNative.q8PreparedFloats(k, n_rows))
    Stream().q8_prepare(wq, prep, k, n_rows).run()
    counts = HipNative.profileOps(op.array(), 1, detail=True)[2]
    assert counts[0] == (1 if tile[2] == 1 else 2) + 1        # activation split, GEMM, and the sum of the shares
    op.run()
    got = dev.download(ob, (m, n))
    assert_close(exp, got, atol=gate(exp), rtol=1e-4, what=f"fp16 GEMM on prepared weights M={m} K={k} N={n} {epilogue}")
    dev.release(xb, ob, wq, prep, *kw_buffers(kw))


def kw_buffers(kw):
    return [v for v in kw.values() if not isinstance(v, bool)]


def test_random_shapes_both_tiles_and_shared_k(dev):
    """Seeded random (M, K, N) over the kernel's whole domain - M not a multiple of 64, K not a multiple of 32, N only a
    multiple of 4 - until each of the three ways the library takes a problem (128-row tiles, 64-row tiles, 64-row tiles
    with K shared by several workgroups) has been exercised twice."""
    rng = np.random.default_rng(20240607)
    seen = {"128": 0, "64": 0, "64 shared": 0}
    tries = 0
    while min(seen.values()) < 2 and tries < 200:
        tries += 1
        m = int(rng.integers(256, 700))
        k = int(rng.integers(64, 6000))
        n = 4 * int(rng.integers(128, 4000))
        tile = HipNative.q8GemmPath(m, k, n)
        if tile == 0:
            continue
        cols = -(-n // 256)
        shared = tile == 64 and -(-m // 64) * cols < 128
        key = "64 shared" if shared else str(tile)
        if seen[key] >= 2:
            continue
        seen[key] += 1
        w = (rng.standard_normal((k, n)) * 0.03).astype(np.float32)
        x = rng.standard_normal((m, k)).astype(np.float32)
        r = rng.standard_normal((m, n)).astype(np.float32)
        wq, deq = quantised(dev, w)
        exp = ref.add(r, ref.matmul(x, deq))
        xb, rb, ob = dev.upload(x), dev.upload(r), dev.alloc(m * n)
        Stream().q8_linear(xb, wq, ob, m, k, n, residual=rb).run()
        got = dev.download(ob, (m, n))
        dev.release(xb, rb, ob, wq)
        assert_close(exp, got, atol=gate(exp), rtol=1e-4, what=f"Q8 linear M={m} K={k} N={n} ({key})")
    assert min(seen.values()) >= 2, seen


def test_rows_spanning_twelve_decades_with_outliers(dev):
    """Each row gets its own power of two before the fp16 split: a row of 1e-6 magnitudes must come out as exact as a
    row of 1e6; inside a row, values 300 times the typical size and values 1e-4 of it share the row's scale."""
    m, k, n = 260, 512, 40960
    assert HipNative.q8GemmPath(m, k, n) == 128
    x = JavaRandom(21).tensor(m, k, 1.0)
    x *= (10.0 ** ((np.arange(m) % 13) - 6)).astype(np.float32)[:, None]
    x[:, 5::97] *= 300.0
    x[:, 7::89] *= 1e-4
    x[17, :] = 0.0                                                # an all-zero row
    x[18, 3] = 0.0
    w = JavaRandom(22).tensor(k, n, 0.02)
    wq, deq = quantised(dev, w)
    exp = ref.matmul(x, deq)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    Stream().q8_linear(xb, wq, ob, m, k, n).run()
    got = dev.download(ob, (m, n))
    dev.release(xb, ob, wq)
    assert not got[17].any()
    # per row: the row's own rms sets the tolerance (the rows differ by twelve decades)
    rms = np.sqrt(np.mean(exp.astype(np.float64) ** 2, axis=1, keepdims=True))
    err = np.abs(got.astype(np.float64) - exp) - 1e-4 * np.abs(exp)
    worst = float(np.max(err / np.maximum(rms, 1e-300)))
    print(f"\n[rows 1e-6 .. 1e6] worst (|err| - 1e-4 |exp|) / row rms = {worst:.2e}")
    assert worst <= 1e-4


@pytest.mark.parametrize("k,n,tile", [(256, 16384, (128, 256, 1)), (256, 14336, (128, 192, 1)), (256, 9216, (64, 256, 1)),
                                      (256, 7680, (64, 192, 1)), (4000, 2052, (64, 256, 4))])   # the last: K shared by four workgroups
@pytest.mark.parametrize("epilogue", ["bias", "bias_gelu", "bias_residual", "residual"])
def test_epilogues(dev, epilogue, k, n, tile):
    m = 384
    assert HipNative.q8GemmTile(m, k, n) == tile
    x = JavaRandom(31).tensor(m, k, 1.0)
    w = JavaRandom(32).tensor(k, n, 0.05)
    b = JavaRandom(33).tensor(1, n, 0.3)
    r = JavaRandom(34).tensor(m, n, 1.0)
    wq, deq = quantised(dev, w)
    exp = ref.matmul(x, deq)
    kw = {}
    if "bias" in epilogue:
        exp = ref.add_row_vector(exp, b)
        kw["bias"] = dev.upload(b)
    if "gelu" in epilogue:
        exp = ref.gelu(exp)
        kw["gelu"] = True
    if "residual" in epilogue:
        exp = ref.add(r, exp)
        kw["residual"] = dev.upload(r)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    Stream().q8_linear(xb, wq, ob, m, k, n, **kw).run()
    got = dev.download(ob, (m, n))
    dev.release(xb, ob, wq, *[v for v in kw.values() if not isinstance(v, bool)])
    assert_close(exp, got, atol=gate(exp), rtol=1e-4, what=f"Q8 linear + {epilogue}")


@pytest.mark.parametrize("dff,tile", [(10368, 128), (4352, 64)])
@pytest.mark.parametrize("norm", ["rms", "layer"])
def test_swiglu_and_norm_prologues(dev, norm, dff, tile):
    """gate/up rows interleaved in one Q8 buffer, SiLU(gate) * up in the epilogue (SwiGLULayer.java:63-70), behind an
    RMSNorm prologue; LayerNorm prologue with a plain bias epilogue (GPT's first MLP projection)."""
    m, d = 300, 320
    x = JavaRandom(41).tensor(m, d, 1.5)
    gamma = (1.0 + JavaRandom(42).tensor(1, d, 0.1)).astype(np.float32)
    xb, gb = dev.upload(x), dev.upload(gamma)
    if norm == "rms":
        assert HipNative.q8GemmPath(m, d, 2 * dff) == tile
        wg, wu = JavaRandom(43).tensor(d, dff, 0.05), JavaRandom(44).tensor(d, dff, 0.05)
        bg, bu = JavaRandom(45).tensor(1, dff, 0.2), JavaRandom(46).tensor(1, dff, 0.2)
        h = ref.rmsnorm(x, gamma)
        exp = ref.multiply(ref.silu(ref.add_row_vector(ref.matmul(h, ref.q8_roundtrip(wg)), bg)),
                           ref.add_row_vector(ref.matmul(h, ref.q8_roundtrip(wu)), bu))
        wgu = dev.alloc(HipNative.q8Floats(d, 2 * dff))
        for w, off in ((wg, 0), (wu, 1)):
            src = dev.upload(w)
            Stream().q8_quantize(src, wgu, d, dff, off, 2, 2 * dff).run()
            dev.release(src)
        ob = dev.alloc(m * dff)
        Stream().q8_linear(xb, wgu, ob, m, d, dff, gamma=gb, bias=dev.upload(bg), bias2=dev.upload(bu), swiglu=True).run()
        got = dev.download(ob, (m, dff))
        dev.release(wgu, ob)
    else:
        n = 2 * dff
        assert HipNative.q8GemmPath(m, d, n) == tile
        beta = JavaRandom(47).tensor(1, d, 0.1)
        w, b = JavaRandom(48).tensor(d, n, 0.05), JavaRandom(49).tensor(1, n, 0.2)
        wq, deq = quantised(dev, w)
        exp = ref.add_row_vector(ref.matmul(ref.layernorm(x, gamma, beta), deq), b)
        ob = dev.alloc(m * n)
        Stream().q8_linear(xb, wq, ob, m, d, n, gamma=gb, beta=dev.upload(beta), bias=dev.upload(b)).run()
        got = dev.download(ob, (m, n))
        dev.release(wq, ob)
    dev.release(xb, gb)
    assert_close(exp, got, atol=gate(exp), rtol=1e-4, what=f"{norm}-norm prologue")


def test_swiglu_on_partial_products_of_a_shared_k(dev):
    """A few-tile gate/up projection over a long K runs as several workgroups per tile; the kernel that adds their
    partial products applies the interleaved biases and the SwiGLU pairing."""
    m, d, dff = 320, 2048, 1024
    assert HipNative.q8GemmTile(m, d, 2 * dff) == (64, 256, 6)
    x = JavaRandom(51).tensor(m, d, 1.0)
    gamma = (1.0 + JavaRandom(52).tensor(1, d, 0.1)).astype(np.float32)
    wg, wu = JavaRandom(53).tensor(d, dff, 0.03), JavaRandom(54).tensor(d, dff, 0.03)
    bg, bu = JavaRandom(55).tensor(1, dff, 0.2), JavaRandom(56).tensor(1, dff, 0.2)
    h = ref.rmsnorm(x, gamma)
    exp = ref.multiply(ref.silu(ref.add_row_vector(ref.matmul(h, ref.q8_roundtrip(wg)), bg)),
                       ref.add_row_vector(ref.matmul(h, ref.q8_roundtrip(wu)), bu))
    wgu = dev.alloc(HipNative.q8Floats(d, 2 * dff))
    for w, off in ((wg, 0), (wu, 1)):
        src = dev.upload(w)
        Stream().q8_quantize(src, wgu, d, dff, off, 2, 2 * dff).run()
        dev.release(src)
    xb, gb, ob = dev.upload(x), dev.upload(gamma), dev.alloc(m * dff)
    bgb, bub = dev.upload(bg), dev.upload(bu)
    Stream().q8_linear(xb, wgu, ob, m, d, dff, gamma=gb, bias=bgb, bias2=bub, swiglu=True).run()
    got = dev.download(ob, (m, dff))
    dev.release(wgu, ob, xb, gb, bgb, bub)
    assert_close(exp, got, atol=gate(exp), rtol=1e-4, what="SwiGLU over shared K")


def test_prepared_weights_give_the_same_bits_and_follow_the_weights(dev):
    m, k, n = 512, 512, 10240
    assert HipNative.q8GemmPath(m, k, n) == 128
    x = JavaRandom(51).tensor(m, k, 1.0)
    w1, w2 = JavaRandom(52).tensor(k, n, 0.02), JavaRandom(53).tensor(k, n, 0.02)
    wq, deq1 = quantised(dev, w1)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    lin = Stream().q8_linear(xb, wq, ob, m, k, n)
    lin.run()
    plain = dev.download(ob, (m, n))
    prep = dev.alloc(HipNative.q8PreparedFloats(k, n))
    Stream().q8_prepare(wq, prep, k, n).run()
    lin.run()
    with_prepared = dev.download(ob, (m, n))
    assert np.array_equal(plain.view(np.int32), with_prepared.view(np.int32))
    # new weights in the same buffer: the copy no longer stands for them
    src = dev.upload(w2)
    Stream().q8_quantize(src, wq, k, n).run()
    lin.run()
    got = dev.download(ob, (m, n))
    exp = ref.matmul(x, ref.q8_roundtrip(w2))
    assert_close(exp, got, atol=gate(exp), rtol=1e-4, what="after re-quantising a prepared weight")
    # prepared again, then the copy is released: back to per-call conversion, same result
    Stream().q8_prepare(wq, prep, k, n).run()
    dev.release(prep)
    lin.run()
    assert np.array_equal(dev.download(ob, (m, n)).view(np.int32), got.view(np.int32))
    with pytest.raises(RuntimeError, match="a buffer of its own"):
        Stream().q8_prepare(wq, wq, k, n).run()
    dev.release(src, wq, xb, ob)


def test_runner_prepared_weight_budgets_give_identical_logits_and_tokens():
    """Whatever a runner may spend on fp16 copies of its weights for the prompt GEMM - every layer, the first two,
    none - the arithmetic is the same: identical logits, bit for bit, and identical tokens; the bytes held follow
    the budget."""
    from deepj_amd import LlamaConfig, LlamaModel, TextGenerator
    cfg = LlamaConfig(vocabSize=512, maxSeqLen=384, dModel=1024, nHeads=16, nLayers=4, dFF=3328)
    assert HipNative.q8GemmPath(320, 1024, 2 * 3328) != 0        # the gate/up projection takes the fp16 GEMM at this size
    prompt = JavaRandom(5).ints(320, 512)
    model = LlamaModel(cfg, 42)
    try:
        full = model.preparedBytes()
        assert full > 0                                          # the warm-up pass prepared every layer
        results, held = {}, {}
        for name, budget in (("all", None), ("two layers", full // 2), ("none", 0), ("all again", None)):
            model.setPreparedBudget(budget)
            assert model.preparedBytes() == 0                    # released; the next long prompt prepares anew
            logits = model.forward(prompt)
            toks = TextGenerator.generate(model, prompt, 8, top_k=1)
            held[name] = model.preparedBytes()
            results[name] = (logits, toks)
        for name in ("two layers", "none", "all again"):
            assert np.array_equal(results[name][0].view(np.int32), results["all"][0].view(np.int32)), name
            assert np.array_equal(results[name][1], results["all"][1]), name
        assert held["none"] == 0 and held["all"] == held["all again"] == full
        assert 0 < held["two layers"] <= full // 2
        with pytest.raises(ValueError, match="budget must be"):
            model.setPreparedBudget(-5)
    finally:
        model.close()


def test_graph_replays_of_the_gemm_match_eager_runs(dev):
    """The three-kernel Q8_LINEAR (split, GEMM on shared K, sum of partial products) and the single-GEMM one captured into
    a HIP graph: every replay, with eager work and synchronisation in between, gives the eager run's bits."""
    for m, k, n in ((512, 5632, 2048), (300, 320, 20736)):
        assert HipNative.q8GemmPath(m, k, n) != 0
        x = JavaRandom(61).tensor(m, k, 1.0)
        w = JavaRandom(62).tensor(k, n, 0.02)
        r = JavaRandom(63).tensor(m, n, 1.0)
        wq, _ = quantised(dev, w)
        xb, rb, ob, scratch = dev.upload(x), dev.upload(r), dev.alloc(m * n), dev.alloc(m * n)
        lin = Stream().q8_linear(xb, wq, ob, m, k, n, residual=rb)
        lin.run()
        eager = dev.download(ob, (m, n))
        graph = HipNative.graphCapture(lin.array())
        try:
            for i in range(3):
                Stream().fill(ob, 0, m * n).fill(scratch, i + 1, m * n).run()
                HipNative.synchronize()
                HipNative.graphLaunch(graph, 1)
                assert np.array_equal(dev.download(ob, (m, n)).view(np.int32), eager.view(np.int32)), f"replay {i}"
        finally:
            HipNative.graphDestroy(graph)
        dev.release(xb, rb, ob, scratch, wq)


def test_graph_with_prepared_weights_is_refused_once_the_weights_change(dev):
    """A graph captured while a prepared copy stood for the weights replays that copy's address: once the weights are
    written again the copy is stale and the replay must be refused, not run on the old weights.  A stream that prepares
    the copy itself rewrites it on every replay and stays valid."""
    m, k, n = 512, 512, 10240
    x = JavaRandom(71).tensor(m, k, 1.0)
    w1, w2 = JavaRandom(72).tensor(k, n, 0.02), JavaRandom(73).tensor(k, n, 0.02)
    wq, _ = quantised(dev, w1)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    prep = dev.alloc(HipNative.q8PreparedFloats(k, n))
    Stream().q8_prepare(wq, prep, k, n).run()
    lin = Stream().q8_linear(xb, wq, ob, m, k, n)
    lin.run()
    first = dev.download(ob, (m, n))
    uses_copy = HipNative.graphCapture(lin.array())
    own_copy = HipNative.graphCapture(Stream().q8_prepare(wq, prep, k, n).q8_linear(xb, wq, ob, m, k, n).array())
    try:
        Stream().fill(ob, 0, m * n).run()
        HipNative.graphLaunch(uses_copy, 1)
        assert np.array_equal(dev.download(ob, (m, n)).view(np.int32), first.view(np.int32))
        src = dev.upload(w2)
        Stream().q8_quantize(src, wq, k, n).run()              # the copy no longer stands for wq
        with pytest.raises(RuntimeError, match="were written after graph"):
            HipNative.graphLaunch(uses_copy, 1)
        lin.run()
        second = dev.download(ob, (m, n))
        assert not np.array_equal(second, first)
        Stream().fill(ob, 0, m * n).run()
        HipNative.graphLaunch(own_copy, 1)                      # converts the new weights, then multiplies
        assert np.array_equal(dev.download(ob, (m, n)).view(np.int32), second.view(np.int32))
    finally:
        HipNative.graphDestroy(uses_copy)
        HipNative.graphDestroy(own_copy)
    dev.release(src, wq, xb, ob, prep)


@pytest.mark.parametrize("m,k,H,hd,norm", [(512, 2048, 32, 64, "rms"), (300, 512, 24, 128, "layer"), (260, 384, 96, 32, None)])
def test_qkv_projection_with_rope_and_cache_append_as_its_epilogue(dev, m, k, H, hd, norm):
    """OP_Q8_LINEAR_ROPE against OP_Q8_LINEAR followed by OP_ROPE_KV_STORE on the same buffers: rotated queries, the
    rows appended to both caches of the layer (and nothing else in them touched), from a position inside the cache."""
    d, max_seq, layers, layer, pos0 = H * hd, 640, 2, 1, 37
    assert HipNative.q8LinearRopeOk(m, k, d)
    x = JavaRandom(71).tensor(m, k, 1.0)
    w = JavaRandom(72).tensor(k, 3 * d, 0.05)
    b = JavaRandom(73).tensor(1, 3 * d, 0.2)
    gamma = (1.0 + JavaRandom(74).tensor(1, k, 0.1)).astype(np.float32)
    beta = JavaRandom(75).tensor(1, k, 0.1)
    cos, sin = ref.rope_tables(hd, max_seq)
    wq, _ = quantised(dev, w)
    xb, bb, gb, beb = dev.upload(x), dev.upload(b), dev.upload(gamma), dev.upload(beta)
    cos_b, sin_b = dev.upload(cos), dev.upload(sin)
    state = dev.upload(np.array([pos0, 0, 0, 0], np.int32))
    kw = {"bias": bb}
    if norm == "rms":
        kw["gamma"] = gb
    elif norm == "layer":
        kw["gamma"], kw["beta"] = gb, beb
    cache_floats = layers * H * max_seq * hd
    results = []
    for fused in (False, True):
        kc, vc, qo = dev.alloc(cache_floats), dev.alloc(cache_floats), dev.alloc(m * d)
        Stream().fill(kc, 0x40400000, cache_floats).fill(vc, 0x40800000, cache_floats).fill(qo, 0, m * d).run()
        if fused:
            Stream().q8_linear_rope(xb, wq, qo, m, k, d, kc, vc, state, cos_b, sin_b, H, hd, max_seq, layer, **kw).run()
        else:
            qkv = dev.alloc(m * 3 * d)
            Stream().q8_linear(xb, wq, qkv, m, k, 3 * d, **kw).rope_kv_store(qkv, qo, kc, vc, state, cos_b, sin_b, m, H, hd, max_seq, layer).run()
            dev.release(qkv)
        results.append((dev.download(qo, (m, d)), dev.download(kc, (layers, H, max_seq, hd)), dev.download(vc, (layers, H, max_seq, hd))))
        dev.release(kc, vc, qo)
    (q0, k0, v0), (q1, k1, v1) = results
    assert np.array_equal(v0, v1)                                         # values are stored as they are
    assert_close(q0, q1, atol=1e-6, rtol=1e-6, what="rotated queries")
    assert_close(k0, k1, atol=1e-6, rtol=1e-6, what="key cache")
    assert np.all(k1[0] == 3.0) and np.all(v1[0] == 4.0)                  # the other layer is untouched
    assert np.all(k1[1][:, :pos0] == 3.0) and np.all(k1[1][:, pos0 + m:] == 3.0)
    assert np.all(v1[1][:, :pos0] == 4.0) and np.all(v1[1][:, pos0 + m:] == 4.0)
    dev.release(xb, bb, gb, beb, cos_b, sin_b, state, wq)


def test_rope_epilogue_is_refused_where_the_fp16_gemm_is_not_taken(dev):
    m, k, H, hd = 64, 256, 4, 64                                           # too few rows for the fp16 GEMM
    d, max_seq = H * hd, 128
    assert not HipNative.q8LinearRopeOk(m, k, d)
    wq, _ = quantised(dev, JavaRandom(76).tensor(k, 3 * d, 0.05))
    cos, sin = ref.rope_tables(hd, max_seq)
    xb, qo = dev.upload(JavaRandom(77).tensor(m, k, 1.0)), dev.alloc(m * d)
    kc, vc = dev.alloc(H * max_seq * hd), dev.alloc(H * max_seq * hd)
    state, cos_b, sin_b = dev.upload(np.zeros(4, np.int32)), dev.upload(cos), dev.upload(sin)
    with pytest.raises(RuntimeError, match="does not run on the fp16 GEMM"):
        Stream().q8_linear_rope(xb, wq, qo, m, k, d, kc, vc, state, cos_b, sin_b, H, hd, max_seq, 0).run()
    with pytest.raises(RuntimeError, match="bad shape"):
        Stream().q8_linear_rope(xb, wq, qo, 512, k, d, kc, vc, state, cos_b, sin_b, H + 1, hd, max_seq, 0).run()


def test_a_shared_k_gemm_prepares_the_next_normalised_gemm_without_changing_a_bit(dev):
    """Two consecutive ops, the second an RMSNorm'd projection of the first one's output: in one stream the first op's
    sum kernel also writes the second's activation planes (one dispatch instead of two); run as two separate streams
    each op does its own part.  Same bits either way, for a plain and a q | k | v + RoPE second op."""
    m, d, dff, H, hd, max_seq = 512, 2048, 1024, 32, 64, 600
    assert HipNative.q8GemmTile(m, d, d)[2] > 1
    x = JavaRandom(81).tensor(m, d, 1.0)
    res = JavaRandom(82).tensor(m, d, 1.0)
    gamma = (1.0 + JavaRandom(83).tensor(1, d, 0.1)).astype(np.float32)
    bias = JavaRandom(84).tensor(1, d, 0.2)
    w1, _ = quantised(dev, JavaRandom(85).tensor(d, d, 0.03))
    w2, _ = quantised(dev, JavaRandom(86).tensor(d, 2 * dff, 0.03))
    w3, _ = quantised(dev, JavaRandom(87).tensor(d, 3 * d, 0.03))
    cos, sin = ref.rope_tables(hd, max_seq)
    xb, rb, gb, bb = dev.upload(x), dev.upload(res), dev.upload(gamma), dev.upload(bias)
    cos_b, sin_b, state = dev.upload(cos), dev.upload(sin), dev.upload(np.array([5, 0, 0, 0], np.int32))
    mid, out, qo = dev.alloc(m * d), dev.alloc(m * dff), dev.alloc(m * d)
    kc, vc = dev.alloc(H * max_seq * hd), dev.alloc(H * max_seq * hd)

    first = Stream().q8_linear(xb, w1, mid, m, d, d, bias=bb, residual=rb)
    second = Stream().q8_linear(mid, w2, out, m, d, dff, gamma=gb, swiglu=True)
    second_rope = Stream().q8_linear_rope(mid, w3, qo, m, d, d, kc, vc, state, cos_b, sin_b, H, hd, max_seq, 0, gamma=gb)

    first.run(); second.run(); second_rope.run()
    want = (dev.download(mid, (m, d)), dev.download(out, (m, dff)), dev.download(qo, (m, d)), dev.download(kc, (H, max_seq, hd)))
    for buf_id, n in ((mid, m * d), (out, m * dff), (qo, m * d)):
        Stream().fill(buf_id, 0, n).run()
    both = Stream()
    both.words = first.words + second.words
    both.run()
    assert np.array_equal(dev.download(mid, (m, d)), want[0]) and np.array_equal(dev.download(out, (m, dff)), want[1])
    _, _, count = HipNative.profileOps(both.array(), 2, detail=True)
    # split, weight conversion, GEMM, sum + next split | weight conversion, GEMM, sum (it shares K too) - alone: 4
    assert list(count) == [4, 3] and list(HipNative.profileOps(second.array(), 2, detail=True)[2]) == [4]
    Stream().fill(mid, 0, m * d).run()
    both.words = first.words + second_rope.words
    both.run()
    assert np.array_equal(dev.download(mid, (m, d)), want[0]) and np.array_equal(dev.download(qo, (m, d)), want[2])
    assert np.array_equal(dev.download(kc, (H, max_seq, hd)), want[3])
    # an op in between, or another gain, and the second op splits its rows itself
    other = dev.upload((gamma * 1.5).astype(np.float32))
    both.words = first.words + Stream().q8_linear(mid, w2, out, m, d, dff, gamma=other, swiglu=True).words
    both.run()
    with_other = dev.download(out, (m, dff))
    Stream().q8_linear(mid, w2, out, m, d, dff, gamma=other, swiglu=True).run()
    assert np.array_equal(dev.download(out, (m, dff)), with_other) and not np.array_equal(with_other, want[1])
