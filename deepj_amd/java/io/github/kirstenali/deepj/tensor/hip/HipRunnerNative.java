package io.github.kirstenali.deepj.tensor.hip;

/**
 * JNI bridge to the native decode driver (the {@code deepj_runner_*} functions of include/deepj_hip.h,
 * wrapped by csrc/deepj_runner_jni.cpp).  A handle owns the Q8 weights, the KV cache and the per-token
 * command stream of one model; every method throws {@link RuntimeException} with the native message on failure.
 * Loaded together with {@link HipNative} (same libraries).
 */
final class HipRunnerNative {

    private HipRunnerNative() {}

    static boolean available() {
        return HipNative.AVAILABLE;
    }

    /** cfg = {kind (0 Llama, 1 DeepSeek, 2 GPT), vocab, maxSeq, dModel, nHeads, nLayers, dFF, qRank, kvRank}. */
    static native long create(int[] cfg, int idBase);

    static native void destroy(long handle);

    /** One parameter in the reference's orientation ({@code [dIn x dOut]} row-major, vectors {@code [1 x n]}). */
    static native void setWeight(long handle, String name, float[] data, int rows, int cols);

    /** Call once after the last {@link #setWeight}: allocates the cache and the activation buffers. */
    static native void finalizeWeights(long handle);

    /** Logits {@code [ids.length x vocab]} of a fresh sequence, row-major (DecoderOnlyModel.forward). */
    static native float[] forward(long handle, int[] ids, int vocab);

    /** TextGenerator.generate on token ids: returns prompt + maxNewTokens ids.  mode 0 eager, 1 graph. */
    static native int[] generate(long handle, int[] prompt, int maxNewTokens, float temperature, int topK, long seed,
                                 int mode);
}
