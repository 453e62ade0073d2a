package io.github.kirstenali.deepj.tensor.hip;

import io.github.kirstenali.deepj.models.CausalLM;
import io.github.kirstenali.deepj.models.TransformerConfig;
import io.github.kirstenali.deepj.models.deepseek.DeepSeekConfig;
import io.github.kirstenali.deepj.models.gpt.GPTConfig;
import io.github.kirstenali.deepj.optimisers.Parameter;
import io.github.kirstenali.deepj.tensor.Tensor;
import io.github.kirstenali.deepj.tokenizers.Tokenizer;

import java.util.ArrayList;
import java.util.List;

/**
 * Fast inference for a trained (or freshly seeded) LlamaModel, DeepSeekModel or GPTModel: the model's parameters
 * are handed once to the native decode driver, which keeps them as Q8 weights next to a device-resident KV cache
 * and replays one fused command stream per token.  {@link #generate} has the semantics of
 * {@code TextGenerator.generate} (same sliding window, same sampling, same java.util.Random draws).
 *
 * <pre>{@code
 * try (HipDecoder dec = HipDecoder.of(model, cfg)) {
 *     String text = dec.generate(tokenizer, prompt, 128, 0.8f, 40, 1234L);
 * }
 * }</pre>
 */
public final class HipDecoder implements AutoCloseable {

    /** Buffer ids of decoders start here, far above anything a ComputeGraph hands out (it restarts at 0). */
    private static int nextIdBase = 1 << 29;

    private final TransformerConfig cfg;
    private long handle;

    private HipDecoder(TransformerConfig cfg, long handle) {
        this.cfg = cfg;
        this.handle = handle;
    }

    public static synchronized HipDecoder of(CausalLM model, TransformerConfig cfg) {
        if (!HipRunnerNative.available()) throw new IllegalStateException("HIP native library is not loaded");
        int kind = cfg instanceof DeepSeekConfig ? 1 : (cfg instanceof GPTConfig ? 2 : 0);
        int qRank = 0, kvRank = 0;
        if (cfg instanceof DeepSeekConfig ds) {
            qRank = ds.qRank();
            kvRank = ds.kvRank();
        }
        int[] words = {kind, cfg.vocabSize(), cfg.maxSeqLen(), cfg.dModel(), cfg.nHeads(), cfg.nLayers(), cfg.dFF(),
                qRank, kvRank};
        long h = HipRunnerNative.create(words, nextIdBase);
        nextIdBase += 1 << 20;
        HipDecoder dec = new HipDecoder(cfg, h);
        try {
            List<String> names = parameterNames(kind, cfg.nLayers());
            List<Parameter> params = model.parameters();
            if (params.size() != names.size())
                throw new IllegalArgumentException("model has " + params.size() + " parameters, expected " + names.size());
            for (int i = 0; i < params.size(); i++) {
                Tensor t = params.get(i).value;
                t.materialize();                                   // the values may still live on a GPU backend
                HipRunnerNative.setWeight(h, names.get(i), t.data, t.rows, t.cols);
            }
            HipRunnerNative.finalizeWeights(h);
        } catch (RuntimeException e) {
            dec.close();
            throw e;
        }
        return dec;
    }

    /** Names in {@code model.parameters()} order (DecoderOnlyModel.parameters, sub-layers {ln1, ln2, attn, mlp}). */
    static List<String> parameterNames(int kind, int nLayers) {
        String[] per = switch (kind) {
            case 1 -> new String[]{"g1", "g2", "wdq", "wuq", "wdkv", "wuk", "wuv", "wo", "wg", "bg", "wu", "bu", "wd", "bd"};
            case 2 -> new String[]{"g1", "be1", "g2", "be2", "wq", "wk", "wv", "wo", "wg", "bg", "wd", "bd"};
            default -> new String[]{"g1", "g2", "wq", "wk", "wv", "wo", "wg", "bg", "wu", "bu", "wd", "bd"};
        };
        List<String> names = new ArrayList<>();
        names.add("emb");
        if (kind == 2) names.add("pos");
        for (int l = 0; l < nLayers; l++)
            for (String w : per) names.add("L" + l + "." + w);
        names.add("gf");
        if (kind == 2) names.add("bf");
        names.add("wlm");
        names.add("blm");
        return names;
    }

    /** Logits {@code [ids.length x vocabSize]} like {@code model.forward(ids)}. */
    public Tensor forward(int[] ids) {
        float[] logits = HipRunnerNative.forward(handle, ids, cfg.vocabSize());
        Tensor out = Tensor.zeros(ids.length, cfg.vocabSize());
        System.arraycopy(logits, 0, out.data, 0, logits.length);
        return out;
    }

    /** {@code TextGenerator.generate(model, tok, cfg, prompt, maxNewTokens, temperature, topK, seed)}. */
    public String generate(Tokenizer tok, String prompt, int maxNewTokens, float temperature, int topK, long seed) {
        if (maxNewTokens < 0) throw new IllegalArgumentException("maxNewTokens must be >= 0");
        if (temperature <= 0f) throw new IllegalArgumentException("temperature must be > 0");
        if (topK < 0) throw new IllegalArgumentException("topK must be >= 0");
        int[] ids = tok.encode(prompt);
        return tok.decode(HipRunnerNative.generate(handle, ids, maxNewTokens, temperature, topK, seed, 1));
    }

    /** The same on token ids; returns prompt followed by the new ids. */
    public int[] generate(int[] promptIds, int maxNewTokens, float temperature, int topK, long seed) {
        return HipRunnerNative.generate(handle, promptIds, maxNewTokens, temperature, topK, seed, 1);
    }

    @Override
    public void close() {
        if (handle != 0) {
            HipRunnerNative.destroy(handle);
            handle = 0;
        }
    }
}
