"""The drop-in path as a whole model: the reference's layer compositions (tests/reference_layers.py, twins of LlamaModel,
LlamaTransformerBlock, RoPEMultiHeadSelfAttention, HeadOps, RotaryEmbedding, RMSNorm1D, SwiGLULayer, Linear,
Embedding, TextGenerator) over Tensor + HipBackend: every tensor op is one of the 42 primitive opcodes recorded by the
lazy ComputeGraph and executed through the five GpuRuntime calls of the C ABI, with the reference's host loops
(head split / merge, RoPE, per-head block copies) in between.  Expected values: the CPU oracle on the same seeded
fp32 weights (nothing is quantised on this path).

Sizes: the reference's own LlamaModelTest model (src/test/java/io/github/kirstenali/deepj/models/llama/
LlamaModelTest.java:18-29: vocab 256, maxSeqLen 16, dModel 32, 4 heads, 2 layers, dFF = defaultDFF(32)) and the
baseline's tiny Llama (vocab 256, dModel 256, 4 layers, 8 heads, dFF 688, maxSeq 256)."""
import numpy as np
import pytest

import reference_layers as dropin
from deepj_amd import HipBackend, HipGpuRuntime, LlamaConfig, Tensor
from oracle import cpu_ref as ref

pytestmark = pytest.mark.gpu


class CountingRuntime(HipGpuRuntime):
    """The five GpuRuntime calls, counted."""

    def __init__(self):
        self.flushes = self.downloads = self.uploads = 0

    def flushOps(self, cmd_stream, length):
        self.flushes += 1
        super().flushOps(cmd_stream, length)

    def downloadBuffer(self, buf_id, out):
        self.downloads += 1
        super().downloadBuffer(buf_id, out)

    def uploadBuffer(self, buf_id, data):
        self.uploads += 1
        super().uploadBuffer(buf_id, data)


@pytest.fixture
def counting_backend():
    rt = CountingRuntime()
    be = HipBackend(rt)
    Tensor.setBackend(be)
    yield rt
    be.releaseResources()


def oracle_for(cfg, seed):
    return ref.Model(vocab=cfg.vocabSize, max_seq=cfg.maxSeqLen, d=cfg.dModel, heads=cfg.nHeads, layers=cfg.nLayers,
                     dff=cfg.dFF, seed=seed)


SMALL = LlamaConfig(vocabSize=256, maxSeqLen=16, dModel=32, nHeads=4, nLayers=2, dFF=LlamaConfig.defaultDFF(32))
C1 = LlamaConfig(vocabSize=256, maxSeqLen=256, dModel=256, nHeads=8, nLayers=4, dFF=688)


@pytest.mark.parametrize("cfg,prompt_len", [(SMALL, 12), (C1, 32)])
def test_llama_forward_through_primitive_opcodes_matches_oracle(counting_backend, cfg, prompt_len):
    rt = counting_backend
    model = dropin.LlamaModel(cfg, 42)
    cpu = oracle_for(cfg, 42)
    try:
        # seeded parameters are the oracle's, bit for bit, in the reference's parameters() order
        assert len(model.parameters()) == 1 + 12 * cfg.nLayers + 1 + 2            # LlamaModelTest.java:104-111
        for name, t in (("emb", model.tokEmb.weight.value), ("wlm", model.lmHead.W.value),
                        (f"L{cfg.nLayers - 1}.wd", model.stack.blocks[-1].mlp.downProj.W.value),
                        ("L0.wq", model.stack.blocks[0].attn.Wq.value)):
            assert np.array_equal(t.data.view(np.int32), cpu.weight(name).view(np.int32)), name
        ids = ref.JavaRandom(7).ints(prompt_len, cfg.vocabSize)
        f0, d0 = rt.flushes, rt.downloads
        logits = model.forward(ids)
        logits.materialize()
        flushes, downloads = rt.flushes - f0, rt.downloads - d0
        exp = cpu.forward(ids)
        err = float(np.max(np.abs(logits.data - exp)))
        print(f"\n[drop-in Llama d{cfg.dModel} L{cfg.nLayers} H{cfg.nHeads}, {prompt_len} rows] logits max-abs err {err:.2e}; "
              f"{flushes} flushes, {downloads} downloads for one forward")
        assert err <= 1e-3
        assert np.array_equal(np.argmax(logits.data, axis=1), np.argmax(exp, axis=1))
        # per block: one flush when Q, K, V are first read on the host, one per head in each of scores, mask and
        # P.V, one for the softmax output; the last flush brings the logits
        H, L = cfg.nHeads, cfg.nLayers
        assert flushes == L * (3 * H + 2) + 1
        assert downloads == L * (3 * H + 4) + 1
    finally:
        cpu.close()


@pytest.mark.parametrize("cfg,prompt_len", [(SMALL, 8), (C1, 32)])
def test_llama_greedy_generation_through_primitive_opcodes(counting_backend, cfg, prompt_len):
    """TextGenerator semantics on the drop-in path: no cache, the window re-runs for every token (and slides past
    maxSeqLen on the small model: 8 + 16 tokens against a window of 16).  16 greedy tokens identical to the oracle."""
    model = dropin.LlamaModel(cfg, 42)
    cpu = oracle_for(cfg, 42)
    try:
        prompt = ref.JavaRandom(7).ints(prompt_len, cfg.vocabSize)
        got = dropin.TextGenerator.generate(model.forward, cfg.maxSeqLen, prompt, 16, temperature=1.0, top_k=1, seed=0)
        exp = cpu.generate(prompt, 16, temperature=1.0, top_k=1, seed=0, use_cache=False)
        assert np.array_equal(got[:prompt_len], prompt)                          # LlamaModelTest.java:120-127
        assert np.array_equal(got, exp), f"first mismatch at {int(np.argmax(got != exp))}"
        sampled = dropin.TextGenerator.generate(model.forward, cfg.maxSeqLen, prompt, 6, temperature=0.7, top_k=4, seed=3)
        assert np.array_equal(sampled, cpu.generate(prompt, 6, temperature=0.7, top_k=4, seed=3, use_cache=False))
    finally:
        cpu.close()


def test_dropin_layers_reject_what_the_reference_rejects(counting_backend):
    with pytest.raises(ValueError, match="dModel must be divisible by nHeads"):
        dropin.MultiHeadSelfAttention(30, 4, True, dropin.JavaRandom(1))
    with pytest.raises(ValueError, match="Token id out of range: 256"):
        dropin.LlamaModel(SMALL, 42).forward([1, 256])
    with pytest.raises(ValueError, match="Expected cols=32"):
        dropin.RMSNorm1D(32).forward(Tensor.zeros(2, 16))
    with pytest.raises(ValueError, match="exceeds maxSeqLen"):
        dropin.RotaryEmbedding(8, 4).apply(Tensor.zeros(10, 8), 5, 2)
    with pytest.raises(ValueError, match="temperature must be > 0"):
        dropin.TextGenerator.generate(lambda ids: None, 16, [1], 1, temperature=0.0)
