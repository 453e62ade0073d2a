"""GPT path (GPTModel.java, GPTTransformerBlock.java, LayerNorm1D.java, FNN.java + GELU, PositionalEmbedding.java)
through the C ABI against the CPU oracle: the two ops the path adds (LAYERNORM, ADD_POSITIONS), the LayerNorm
prologue and GELU epilogue of the Q8 linear in its matvec (M = 1) and GEMM (M > 1) forms, and the model end to
end - prompt logits within 1e-3 max-abs, greedy ids identical over 64 tokens - on identical seeded weights with
the oracle run on the dequantised Q8 matrices."""
import numpy as np
import pytest

from deepj_amd import GPTConfig, GPTModel, HipNative, ModelSerializer, TextGenerator, parameter_names
from deepj_amd.fused import DeviceBuffers, Stream
from oracle import cpu_ref as ref
from gpu_util import assert_close

pytestmark = pytest.mark.gpu


def gaussian(rows, cols, seed, scale):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((rows, cols)) * scale).astype(np.float32)


@pytest.fixture
def dev():
    d = DeviceBuffers()
    yield d
    d.release_all()


def quantize_on_device(dev, w):
    k, n = w.shape
    src = dev.upload(w)
    dst = dev.alloc(HipNative.q8Floats(k, n))
    Stream().q8_quantize(src, dst, k, n, 0, 1, n).run()
    dev.release(src)
    return dst


@pytest.mark.parametrize("rows,cols", [(1, 2048), (5, 33), (37, 4096), (3, 1), (260, 64)])
def test_layernorm_op_matches_oracle(dev, rows, cols):
    x = gaussian(rows, cols, 1, 1.5) + np.float32(0.7)
    x[0] *= np.float32(1e-3)                                 # a row whose variance is of the order of eps
    g, b = 1.0 + gaussian(1, cols, 2, 0.3), gaussian(1, cols, 3, 0.5)
    xb, gb, bb, ob = dev.upload(x), dev.upload(g), dev.upload(b), dev.alloc(rows * cols)
    Stream().layernorm(xb, gb, bb, ob, rows, cols).run()
    assert_close(ref.layernorm(x, g, b), dev.download(ob, (rows, cols)), atol=2e-5, rtol=1e-4,
                 what=f"layernorm {rows}x{cols}")


def test_add_positions_op(dev):
    d, max_seq, rows = 48, 10, 4
    x, table = gaussian(rows, d, 4, 1.0), gaussian(max_seq, d, 5, 1.0)
    xb, tb = dev.upload(x), dev.upload(table)
    state = dev.upload(np.array([3, 0, 0, 0], np.int32))
    Stream().add_positions(xb, tb, state, rows, d, max_seq).run()
    assert np.array_equal(dev.download(xb, (rows, d)), ref.add(x, table[3:7]))
    # rows that would sit beyond the table are poisoned, not read out of bounds
    dev.write(state, np.array([8, 0, 0, 0], np.int32))
    dev.write(xb, x)
    Stream().add_positions(xb, tb, state, rows, d, max_seq).run()
    got = dev.download(xb, (rows, d))
    assert np.array_equal(got[:2], ref.add(x[:2], table[8:10])) and np.all(np.isnan(got[2:]))


def gpt_linear_case(dev, m, k, n, *, layernorm=False, gelu=False, bias=True, residual=False, seed=0):
    w = gaussian(k, n, seed + 1, 0.05)
    x = gaussian(m, k, seed + 2, 1.0) + np.float32(0.25)
    wq = quantize_on_device(dev, w)
    xb, ob = dev.upload(x), dev.alloc(m * n)
    kw, h = {}, x
    if layernorm:
        g, be = 1.0 + gaussian(1, k, seed + 3, 0.2), gaussian(1, k, seed + 4, 0.3)
        kw.update(gamma=dev.upload(g), beta=dev.upload(be))
        h = ref.layernorm(x, g, be)
    exp = ref.matmul(h, ref.q8_roundtrip(w))
    if bias:
        b = gaussian(1, n, seed + 5, 0.5)
        kw["bias"] = dev.upload(b)
        exp = ref.add_row_vector(exp, b)
    if gelu:
        exp = ref.gelu(exp)
    if residual:
        r = gaussian(m, n, seed + 6, 1.0)
        kw["residual"] = dev.upload(r)
        exp = ref.add(r, exp)
    Stream().q8_linear(xb, wq, ob, m, k, n, gelu=gelu, **kw).run()
    return exp, dev.download(ob, (m, n))


@pytest.mark.parametrize("m", [1, 7, 130])
@pytest.mark.parametrize("k,n", [(2048, 768), (688, 256), (30, 17), (4096, 300)])
def test_q8_linear_layernorm_prologue(dev, m, k, n):
    exp, got = gpt_linear_case(dev, m, k, n, layernorm=True, seed=20)
    scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
    assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what=f"layernorm+linear m={m} {k}x{n}")


@pytest.mark.parametrize("m", [1, 9, 200])
def test_q8_linear_gelu_epilogue(dev, m):
    for k, n, flags in [(512, 1024, dict(gelu=True)), (256, 130, dict(gelu=True, layernorm=True)),
                        (64, 40, dict(gelu=True, residual=True, bias=False)),
                        (250, 5000, dict(gelu=True))]:                 # K not a multiple of 4, many outputs
        exp, got = gpt_linear_case(dev, m, k, n, seed=30, **flags)
        scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
        assert_close(exp, got, atol=1e-4 * scale, rtol=1e-4, what=f"gelu m={m} {k}x{n} {flags}")


def test_q8_linear_rejects_conflicting_flags(dev):
    from deepj_amd import opcodes as op
    ids = [dev.alloc(64) for _ in range(3)]
    w = quantize_on_device(dev, gaussian(32, 2, 1, 0.1))
    for flags in (op.LIN_SWIGLU | op.LIN_GELU, op.LIN_SWIGLU | op.LIN_LAYERNORM, op.LIN_RMSNORM | op.LIN_LAYERNORM, 64):
        with pytest.raises(RuntimeError, match="OP_Q8_LINEAR"):
            Stream().emit(op.OP_Q8_LINEAR, ids[0], w, ids[1], 1, 32, 1, flags, ids[2], -1, ids[2], -1).run()


# ── the model ────────────────────────────────────────────────────────────────

G1 = GPTConfig(vocabSize=256, maxSeqLen=256, dModel=256, nHeads=8, nLayers=4, dFF=1024)


def oracle_gpt(cfg, seed):
    m = ref.Model(vocab=cfg.vocabSize, max_seq=cfg.maxSeqLen, d=cfg.dModel, heads=cfg.nHeads, layers=cfg.nLayers,
                  dff=cfg.dFF, seed=seed, gpt=True, init_scale=cfg.initScale)
    m.q8_roundtrip()
    return m


@pytest.fixture(scope="module")
def g1():
    ref.set_threads(ref.default_threads())
    # initScale 1: with the default 0.2 every gain is 0.2 and the logits of a random model shrink to ~1e-3,
    # which would make the absolute logit gate vacuous (the default scale has its own test below)
    cfg = GPTConfig(G1.vocabSize, G1.maxSeqLen, G1.dModel, G1.nHeads, G1.nLayers, G1.dFF, initScale=1.0)
    gpu, cpu = GPTModel(cfg, 42), oracle_gpt(cfg, 42)
    yield gpu, cpu
    gpu.close()
    ref.set_threads(1)


def test_gpt_prompt_logits_match_oracle(g1):
    gpu, cpu = g1
    prompt = ref.JavaRandom(7).ints(32, 256)
    got, exp = gpu.forward(prompt), cpu.forward(prompt)
    assert float(np.max(np.abs(exp))) > 0.5                  # the gate below is not vacuous
    err = float(np.max(np.abs(got - exp)))
    assert err <= 1e-3, f"logits max-abs error {err}"
    assert np.array_equal(np.argmax(got, axis=1), np.argmax(exp, axis=1))


def test_gpt_greedy_64_tokens_identical_to_oracle(g1):
    gpu, cpu = g1
    prompt = ref.JavaRandom(7).ints(32, 256)
    exp, exp_logits = cpu.generate(prompt, 64, top_k=1, use_cache=True, return_logits=True)
    srt = np.sort(exp_logits, axis=1)
    gap = float(np.min(srt[:, -1] - srt[:, -2]))
    print(f"\n[GPT] min top-1/top-2 logit gap over 64 steps = {gap:.4f}")
    for kw in (dict(use_graph=True), dict(use_graph=False)):
        got = TextGenerator.generate(gpu, prompt, 64, top_k=1, **kw)
        assert np.array_equal(got, exp), f"{kw}: first mismatch at {int(np.argmax(got != exp))}"
        assert float(np.max(np.abs(gpu.lastLogits() - exp_logits[-1]))) <= 1e-3


def test_gpt_decode_row_equals_prefill_row_and_positions_advance(g1):
    gpu, cpu = g1
    ids = ref.JavaRandom(11).ints(20, 256)
    full = gpu.forward(ids)
    gpu.reset()
    gpu.prefill(ids[:12], choose_next=False)
    gpu.prefill(ids[12:19], choose_next=False)             # second chunk starts at position 12
    gpu.step(int(ids[19]))
    assert float(np.max(np.abs(gpu.lastLogits() - full[19]))) <= 2e-4
    # sampled generation draws exactly as TextGenerator does
    exp = cpu.generate(ids[:8], 12, temperature=0.8, top_k=5, seed=123, use_cache=True)
    assert np.array_equal(TextGenerator.generate(gpu, ids[:8], 12, temperature=0.8, top_k=5, seed=123), exp)


def test_gpt_default_init_scale_and_seeded_weights(tmp_path):
    """new GPTModel(cfg, seed) with the default initScale 0.2: logits are tiny, so the comparison is relative."""
    cfg = GPTConfig(vocabSize=96, maxSeqLen=32, dModel=64, nHeads=2, nLayers=2, dFF=160)
    assert cfg.initScale == pytest.approx(0.2) and cfg.gradClipNorm == 1.0        # GPTModelTest.java:13-17
    gpu, cpu = GPTModel(cfg, 1234), oracle_gpt(cfg, 1234)
    try:
        ids = ref.JavaRandom(5).ints(17, 96)
        got, exp = gpu.forward(ids), cpu.forward(ids)
        scale = float(np.max(np.abs(exp)))
        assert float(np.max(np.abs(got - exp))) <= 1e-4 * max(scale, 1e-6) + 1e-7, (scale, float(np.max(np.abs(got - exp))))
        # a checkpoint in the reference's parameter order loads into an unseeded model and gives the same logits
        raw = ref.Model(vocab=96, max_seq=32, d=64, heads=2, layers=2, dff=160, seed=1234, gpt=True)
        path = tmp_path / "gpt.bin"
        ModelSerializer.save([raw.weight(n) for n in raw.weight_names()], path)
        assert raw.weight_names() == parameter_names(cfg)
        loaded = GPTModel(cfg, None)
        try:
            ModelSerializer.load(loaded, path)
            assert np.array_equal(loaded.forward(ids), got)
        finally:
            loaded.close()
    finally:
        gpu.close()


def test_gpt_edges():
    cfg = GPTConfig(vocabSize=40, maxSeqLen=12, dModel=64, nHeads=2, nLayers=1, dFF=96, initScale=1.0)
    gpu, cpu = GPTModel(cfg, 3), oracle_gpt(cfg, 3)
    try:
        with pytest.raises(ValueError, match="exceeds maxSeqLen"):      # PositionalEmbedding.java:27
            gpu.forward(np.zeros(13, np.int32))
        with pytest.raises(ValueError, match="Token id out of range"):
            gpu.forward([0, 40])
        ids = ref.JavaRandom(2).ints(12, 40)
        assert float(np.max(np.abs(gpu.forward(ids) - cpu.forward(ids)))) <= 1e-3      # the whole table of positions
        assert float(np.max(np.abs(gpu.forward(ids[:1]) - cpu.forward(ids[:1])))) <= 1e-3
        # fill the cache to its last position: prompt 4 + 8 generated
        exp = cpu.generate(ids[:4], 8, top_k=1, use_cache=True)
        assert np.array_equal(TextGenerator.generate(gpu, ids[:4], 8, top_k=1), exp)
    finally:
        gpu.close()
    for bad in (dict(initScale=0.0), dict(initScale=float("nan")), dict(gradClipNorm=0.0), dict(gradClipNorm=float("nan"))):
        with pytest.raises(ValueError):                                   # GPTModelTest.java:35-45
            GPTConfig(11, 8, 4, 2, 1, 8, **bad)
    for args in ((0, 8, 4, 2, 1, 8), (11, 0, 4, 2, 1, 8), (11, 8, 0, 2, 1, 8), (11, 8, 4, 0, 1, 8), (11, 8, 4, 2, 0, 8),
                 (11, 8, 4, 2, 1, 0), (11, 8, 5, 2, 1, 8)):
        with pytest.raises(ValueError):                                   # GPTModelTest.java:47-63
            GPTConfig(*args)
