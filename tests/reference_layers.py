"""Test scaffolding, not part of the library: the drop-in path as a model - Python twins of the reference's layer COMPOSITIONS, written over Tensor exactly as
the Java classes are, so that with Tensor.setBackend(HipBackend()) a whole LlamaModel forward runs through the 42
primitive opcodes, the lazy ComputeGraph and the five GpuRuntime calls - the way an unmodified DeepJ model would.

Nothing here is fused or cached: head split / merge, RoPE, the per-head score, mask and value products and the
block copies run on the host between flushes, as in the reference
(src/main/java/io/github/kirstenali/deepj/layers/transformer/attention/HeadOps.java:33-140), which costs
3 * nHeads + 2 flushes and 3 * nHeads + 4 downloads per block, and every generated token re-runs the whole context
(models/TextGenerator.java:91-100).  This is the correctness surface of the backend; deepj_amd.models holds the
fast path.

Classes and methods keep the reference's names; file:line citations are relative to
src/main/java/io/github/kirstenali/deepj/.
"""
from __future__ import annotations

import math

import numpy as np

from deepj_amd.models import JavaRandom, LlamaConfig
from deepj_amd.tensor import Tensor


class Parameter:
    """optim/Parameter.java: a value and its gradient accumulator."""

    def __init__(self, value: Tensor):
        self.value = value
        self.grad = Tensor.zeros(value.rows, value.cols)


class Linear:
    """layers/Linear.java:13-36: y = x.W + b, W [dIn x dOut] from Tensor.random, b zeros."""

    def __init__(self, d_in: int, d_out: int, rnd: JavaRandom):
        self.dIn, self.dOut = d_in, d_out
        self.W = Parameter(Tensor.random(d_in, d_out, rnd))
        self.b = Parameter(Tensor.zeros(1, d_out))

    def forward(self, x: Tensor) -> Tensor:
        if x.cols != self.dIn:
            raise ValueError(f"Expected input cols={self.dIn} got {x.cols}")
        return x.matmul(self.W.value).addRowVector(self.b.value)

    def parameters(self): return [self.W, self.b]


class RMSNorm1D:
    """layers/transformer/norm/RMSNorm1D.java:30-57: six backend ops, EPS = 1e-6f."""
    EPS = 1e-6

    def __init__(self, dim: int):
        if dim <= 0:
            raise ValueError("dim must be > 0")
        self.dim = dim
        self.gamma = Parameter(Tensor.ones(1, dim))

    def forward(self, x: Tensor) -> Tensor:
        if x.cols != self.dim:
            raise ValueError(f"Expected cols={self.dim} got {x.cols}")
        mean_sq = x.multiply(x).meanAlongRows()
        rms = mean_sq.addScalar(self.EPS).sqrt()
        x_hat = x.divideBroadcastCols(rms)
        return x_hat.multiplyBroadcastRows(self.gamma.value)

    def parameters(self): return [self.gamma]


class SiLU:
    """activations/SiLU.java:20-24."""

    def forward(self, x: Tensor) -> Tensor:
        return x.multiply(x.sigmoidActivation())


class SwiGLULayer:
    """layers/transformer/SwiGLULayer.java:56-70: down(SiLU(gate(x)) * up(x)); the Linears draw gate, up, down in order."""

    def __init__(self, d_model: int, d_ff: int, rnd: JavaRandom):
        if d_model <= 0:
            raise ValueError("dModel must be > 0")
        if d_ff <= 0:
            raise ValueError("dFF must be > 0")
        self.gateProj = Linear(d_model, d_ff, rnd)
        self.upProj = Linear(d_model, d_ff, rnd)
        self.downProj = Linear(d_ff, d_model, rnd)
        self.silu = SiLU()

    def forward(self, x: Tensor) -> Tensor:
        gate = self.gateProj.forward(x)
        up = self.upProj.forward(x)
        fused = self.silu.forward(gate).multiply(up)
        return self.downProj.forward(fused)

    def parameters(self): return self.gateProj.parameters() + self.upProj.parameters() + self.downProj.parameters()


class RotaryEmbedding:
    """transformer/embeddings/RotaryEmbedding.java:52-122: tables via float64 cast to float, pairs (2i, 2i+1),
    rotation on the host after a forced materialize."""

    def __init__(self, head_dim: int, max_seq_len: int):
        if head_dim <= 0 or head_dim % 2 != 0:
            raise ValueError("headDim must be a positive even number")
        if max_seq_len <= 0:
            raise ValueError("maxSeqLen must be > 0")
        self.headDim, self.maxSeqLen, self.halfDim = head_dim, max_seq_len, head_dim // 2
        self.cosTable = np.empty((max_seq_len, self.halfDim), dtype=np.float32)
        self.sinTable = np.empty((max_seq_len, self.halfDim), dtype=np.float32)
        for pos in range(max_seq_len):
            for i in range(self.halfDim):
                expo = np.float32(np.float32(2.0) * np.float32(i)) / np.float32(head_dim)
                theta = np.float32(pos / math.pow(float(np.float32(10000.0)), float(expo)))
                self.cosTable[pos, i] = np.float32(math.cos(float(theta)))
                self.sinTable[pos, i] = np.float32(math.sin(float(theta)))

    def apply(self, t: Tensor, seq_len: int, n_heads: int) -> Tensor:
        if seq_len > self.maxSeqLen:
            raise ValueError(f"seqLen {seq_len} exceeds maxSeqLen {self.maxSeqLen}")
        t.materialize()
        result = Tensor.zeros(t.rows, t.cols)
        cos, sin = self.cosTable[:seq_len], self.sinTable[:seq_len]
        for h in range(n_heads):                                     # rows h * seqLen + pos
            rows = t.data[h * seq_len:(h + 1) * seq_len]
            x0, x1 = rows[:, 0::2], rows[:, 1::2]
            out = result.data[h * seq_len:(h + 1) * seq_len]
            out[:, 0::2] = x0 * cos - x1 * sin                       # fp32 products and sums, unfused like the JVM's
            out[:, 1::2] = x0 * sin + x1 * cos
        return result


class HeadOps:
    """layers/transformer/attention/HeadOps.java:33-140: flat-array head reshapes and the per-head attention loops."""
    _mask_cache: dict[int, Tensor] = {}

    @staticmethod
    def splitHeads(t: Tensor, seq_len: int, n_heads: int, head_dim: int, d_model: int) -> Tensor:
        t.materialize()
        out = Tensor(n_heads * seq_len, head_dim)
        for h in range(n_heads):
            out.data[h * seq_len:(h + 1) * seq_len] = t.data[:seq_len, h * head_dim:(h + 1) * head_dim]
        return out

    @staticmethod
    def mergeHeads(t: Tensor, seq_len: int, n_heads: int, head_dim: int, d_model: int) -> Tensor:
        t.materialize()
        out = Tensor(seq_len, d_model)
        for h in range(n_heads):
            out.data[:, h * head_dim:(h + 1) * head_dim] = t.data[h * seq_len:(h + 1) * seq_len]
        return out

    @staticmethod
    def extractBlock(t: Tensor, row_start: int, num_rows: int, num_cols: int) -> Tensor:
        t.materialize()
        block = Tensor(num_rows, num_cols)
        block.data[:] = t.data[row_start:row_start + num_rows, :num_cols]
        return block

    @staticmethod
    def insertBlock(target: Tensor, block: Tensor, row_start: int, num_rows: int, num_cols: int) -> None:
        block.materialize()
        target.data[row_start:row_start + num_rows, :num_cols] = block.data

    @staticmethod
    def scaledDotProductScores(qh, kh, n_heads, seq_len, head_dim, scale) -> Tensor:
        out = Tensor(n_heads * seq_len, seq_len)
        for h in range(n_heads):
            q = HeadOps.extractBlock(qh, h * seq_len, seq_len, head_dim)
            k = HeadOps.extractBlock(kh, h * seq_len, seq_len, head_dim)
            s = q.matmul(k.transpose())
            s.multiplyScalarInPlace(scale)
            s.materialize()
            HeadOps.insertBlock(out, s, h * seq_len, seq_len, seq_len)
        return out

    @staticmethod
    def applyCausalMask(scores: Tensor, n_heads: int, seq_len: int) -> Tensor:
        mask = HeadOps._mask_cache.get(seq_len)
        if mask is None:
            mask = Tensor.causalMask(seq_len)                      # -1e9f above the diagonal, additive
            HeadOps._mask_cache[seq_len] = mask
        out = Tensor(n_heads * seq_len, seq_len)
        for h in range(n_heads):
            block = HeadOps.extractBlock(scores, h * seq_len, seq_len, seq_len)
            masked = block.add(mask)
            masked.materialize()
            HeadOps.insertBlock(out, masked, h * seq_len, seq_len, seq_len)
        return out

    @staticmethod
    def applyAttentionToValues(attn_prob, vh, n_heads, seq_len, head_dim) -> Tensor:
        out = Tensor(n_heads * seq_len, head_dim)
        for h in range(n_heads):
            a = HeadOps.extractBlock(attn_prob, h * seq_len, seq_len, seq_len)
            v = HeadOps.extractBlock(vh, h * seq_len, seq_len, head_dim)
            y = a.matmul(v)
            y.materialize()
            HeadOps.insertBlock(out, y, h * seq_len, seq_len, head_dim)
        return out


class MultiHeadSelfAttention:
    """layers/transformer/attention/MultiHeadSelfAttention.java:36-86: bare parameters Wq, Wk, Wv, Wo (no bias),
    scale = (float)(1 / sqrt(headDim)) applied after the product."""

    def __init__(self, d_model: int, n_heads: int, causal_mask: bool, rnd: JavaRandom):
        if d_model % n_heads != 0:
            raise ValueError("dModel must be divisible by nHeads")
        self.dModel, self.nHeads, self.headDim, self.causalMask = d_model, n_heads, d_model // n_heads, causal_mask
        self.scale = float(np.float32(1.0 / math.sqrt(self.headDim)))
        self.Wq = Parameter(Tensor.random(d_model, d_model, rnd))
        self.Wk = Parameter(Tensor.random(d_model, d_model, rnd))
        self.Wv = Parameter(Tensor.random(d_model, d_model, rnd))
        self.Wo = Parameter(Tensor.random(d_model, d_model, rnd))

    def transformQueryKey(self, heads: Tensor, seq_len: int) -> Tensor:
        return heads

    def forward(self, x: Tensor) -> Tensor:
        if x.cols != self.dModel:
            raise ValueError(f"Expected input cols={self.dModel} got {x.cols}")
        S, H, hd, d = x.rows, self.nHeads, self.headDim, self.dModel
        q, k, v = x.matmul(self.Wq.value), x.matmul(self.Wk.value), x.matmul(self.Wv.value)
        qh, kh, vh = (HeadOps.splitHeads(t, S, H, hd, d) for t in (q, k, v))
        qh, kh = self.transformQueryKey(qh, S), self.transformQueryKey(kh, S)
        scores = HeadOps.scaledDotProductScores(qh, kh, H, S, hd, self.scale)
        if self.causalMask:
            scores = HeadOps.applyCausalMask(scores, H, S)
        attn_prob = scores.softmaxRows()                             # activations/Softmax.java:16-19
        out_h = HeadOps.applyAttentionToValues(attn_prob, vh, H, S, hd)
        merged = HeadOps.mergeHeads(out_h, S, H, hd, d)
        return merged.matmul(self.Wo.value)

    def parameters(self): return [self.Wq, self.Wk, self.Wv, self.Wo]


class RoPEMultiHeadSelfAttention(MultiHeadSelfAttention):
    """layers/transformer/attention/RoPEMultiHeadSelfAttention.java:40-58."""

    def __init__(self, d_model, n_heads, causal_mask, rope: RotaryEmbedding, rnd: JavaRandom):
        super().__init__(d_model, n_heads, causal_mask, rnd)
        if rope is None:
            raise ValueError("rope must not be null")
        self.rope = rope

    def transformQueryKey(self, heads: Tensor, seq_len: int) -> Tensor:
        return self.rope.apply(heads, seq_len, self.nHeads)


class LlamaTransformerBlock:
    """layers/transformer/blocks/LlamaTransformerBlock.java:34-53: pre-norm residual block; parameters in the
    order ln1, ln2, attn, mlp."""

    def __init__(self, d_model, n_heads, d_ff, max_seq_len, rnd: JavaRandom):
        rope = RotaryEmbedding(d_model // n_heads, max_seq_len)
        self.ln1, self.ln2 = RMSNorm1D(d_model), RMSNorm1D(d_model)
        self.attn = RoPEMultiHeadSelfAttention(d_model, n_heads, True, rope, rnd)
        self.mlp = SwiGLULayer(d_model, d_ff, rnd)

    def forward(self, x: Tensor) -> Tensor:
        x2 = x.add(self.attn.forward(self.ln1.forward(x)))
        return x2.add(self.mlp.forward(self.ln2.forward(x2)))

    def parameters(self):
        return self.ln1.parameters() + self.ln2.parameters() + self.attn.parameters() + self.mlp.parameters()


class TransformerStack:
    """transformer/TransformerStack.java:20-35."""

    def __init__(self, blocks):
        if not blocks:
            raise ValueError("blocks must be non-empty")
        self.blocks = list(blocks)

    def forward(self, x: Tensor) -> Tensor:
        for b in self.blocks:
            x = b.forward(x)
        return x

    def parameters(self): return [p for b in self.blocks for p in b.parameters()]


class Embedding:
    """transformer/embeddings/Embedding.java:21-34: host gather of table rows (Tensor.sliceRows)."""

    def __init__(self, vocab_size: int, d_model: int, rnd: JavaRandom):
        self.vocabSize, self.dModel = vocab_size, d_model
        self.weight = Parameter(Tensor.random(vocab_size, d_model, rnd))

    def forward(self, ids) -> Tensor:
        for i in ids:
            if i < 0 or i >= self.vocabSize:
                raise ValueError(f"Token id out of range: {int(i)}")
        return Tensor.sliceRows(self.weight.value, [int(i) for i in ids], self.dModel)

    def parameters(self): return [self.weight]


class LlamaModel:
    """models/llama/LlamaModel.java:27-42 + models/DecoderOnlyModel.java:58-64: embedding from Random(seed), the block
    stack from its own Random(seed) (transformer/LlamaTransformerBuilder.java:45-55), the head from Random(seed + 1)."""

    def __init__(self, cfg: LlamaConfig, seed: int):
        self.cfg = cfg
        self.tokEmb = Embedding(cfg.vocabSize, cfg.dModel, JavaRandom(seed))
        stack_rnd = JavaRandom(seed)
        self.stack = TransformerStack([LlamaTransformerBlock(cfg.dModel, cfg.nHeads, cfg.dFF, cfg.maxSeqLen, stack_rnd)
                                       for _ in range(cfg.nLayers)])
        self.normF = RMSNorm1D(cfg.dModel)
        self.lmHead = Linear(cfg.dModel, cfg.vocabSize, JavaRandom(seed + 1))

    def forward(self, input_ids) -> Tensor:
        x = self.tokEmb.forward(input_ids)
        x = self.stack.forward(x)
        x = self.normF.forward(x)
        return self.lmHead.forward(x)                                # logits [seqLen x vocabSize]

    def parameters(self):
        return self.tokEmb.parameters() + self.stack.parameters() + self.normF.parameters() + self.lmHead.parameters()


class TextGenerator:
    """models/TextGenerator.java:66-181 on token ids: every token re-runs the window through `forwarder`."""

    @staticmethod
    def generate(forwarder, max_seq_len: int, prompt_ids, max_new_tokens: int, temperature: float = 1.0,
                 top_k: int = 1, seed: int = 0) -> np.ndarray:
        if max_new_tokens < 0:
            raise ValueError("maxNewTokens must be >= 0")
        if not temperature > 0.0:
            raise ValueError("temperature must be > 0")
        if top_k < 0:
            raise ValueError("topK must be >= 0")
        rnd = JavaRandom(seed)
        ids = [int(i) for i in prompt_ids]
        for _ in range(max_new_tokens):
            context = ids[-max_seq_len:] if len(ids) > max_seq_len else ids
            logits = forwarder(context)
            logits.materialize()
            ids.append(TextGenerator.sampleFromLogits(logits.data[logits.rows - 1], temperature, top_k, rnd))
        return np.asarray(ids, dtype=np.int32)

    @staticmethod
    def sampleFromLogits(logits: np.ndarray, temperature: float, top_k: int, rnd: JavaRandom) -> int:
        order = np.argsort(-logits.astype(np.float32), kind="stable")          # ties: lowest index first (:163-170)
        k = len(logits) if top_k == 0 else min(top_k, len(logits))
        idx = order[:k]
        t = np.float32(temperature)
        scaled = logits[idx].astype(np.float32) / t
        mx = np.float32(scaled.max())
        probs = np.exp((scaled - mx).astype(np.float64)).astype(np.float32)     # (float) Math.exp(l / T - max)
        total = np.float32(0.0)
        for p in probs:
            total = np.float32(total + p)
        probs = probs / total
        r = np.float32(rnd.nextFloat())
        cum = np.float32(0.0)
        for i, p in enumerate(probs):
            cum = np.float32(cum + p)
            if r <= cum:
                return int(idx[i])
        return int(idx[-1])
