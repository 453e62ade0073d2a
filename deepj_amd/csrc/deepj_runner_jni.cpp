// JNI shim for io.github.kirstenali.deepj.tensor.hip.HipRunnerNative: one wrapper per deepj_runner_* function of
// include/deepj_hip.h that the Java facade (HipDecoder) uses.  Same conventions as deepj_hip_jni.cpp: input
// arrays released with JNI_ABORT, failures raised as java.lang.RuntimeException with the native message.
//
// Build (needs a JDK for jni.h; not part of the default build because the build image has none) - both shims
// go into the one library HipNative loads:
//   hipcc -shared -fPIC -I$JAVA_HOME/include -I$JAVA_HOME/include/linux \
//         deepj_hip_jni.cpp deepj_runner_jni.cpp -L.. -ldeepj_hip -o libdeepj_hip_jni.so
#include <jni.h>

#include <string>
#include <vector>

#include "../../include/deepj_hip.h"

namespace {

void throw_runtime(JNIEnv *env, const char *msg) {
    jclass cls = env->FindClass("java/lang/RuntimeException");
    if (cls != nullptr) env->ThrowNew(cls, msg);
}

// true when the call failed (an exception is then pending)
bool failed(JNIEnv *env, void *runner, int rc) {
    if (rc == 0) return false;
    throw_runtime(env, deepj_runner_last_error(runner));
    return true;
}

void *ptr(jlong handle) { return reinterpret_cast<void *>(static_cast<intptr_t>(handle)); }

}  // namespace

extern "C" {

JNIEXPORT jlong JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipRunnerNative_create(JNIEnv *env, jclass,
                                                                                         jintArray cfg_arr,
                                                                                         jint id_base) {
    if (env->GetArrayLength(cfg_arr) != 9) {
        throw_runtime(env, "runner config needs 9 words");
        return 0;
    }
    jint *cfg = env->GetIntArrayElements(cfg_arr, nullptr);
    void *r = deepj_runner_create(reinterpret_cast<const int32_t *>(cfg), id_base);
    env->ReleaseIntArrayElements(cfg_arr, cfg, JNI_ABORT);
    if (r == nullptr) throw_runtime(env, "invalid model configuration");
    return static_cast<jlong>(reinterpret_cast<intptr_t>(r));
}

JNIEXPORT void JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipRunnerNative_destroy(JNIEnv *, jclass, jlong h) {
    deepj_runner_destroy(ptr(h));
}

JNIEXPORT void JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipRunnerNative_setWeight(
    JNIEnv *env, jclass, jlong h, jstring name_str, jfloatArray data_arr, jint rows, jint cols) {
    if ((jlong)env->GetArrayLength(data_arr) < (jlong)rows * cols) {
        throw_runtime(env, "setWeight: array shorter than rows * cols");
        return;
    }
    const char *name = env->GetStringUTFChars(name_str, nullptr);
    jfloat *data = env->GetFloatArrayElements(data_arr, nullptr);
    int rc = deepj_runner_set_weight(ptr(h), name, data, rows, cols);
    env->ReleaseFloatArrayElements(data_arr, data, JNI_ABORT);
    env->ReleaseStringUTFChars(name_str, name);
    failed(env, ptr(h), rc);
}

JNIEXPORT void JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipRunnerNative_finalizeWeights(JNIEnv *env, jclass,
                                                                                                  jlong h) {
    failed(env, ptr(h), deepj_runner_finalize(ptr(h)));
}

JNIEXPORT jfloatArray JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipRunnerNative_forward(
    JNIEnv *env, jclass, jlong h, jintArray ids_arr, jint vocab) {
    jint n = env->GetArrayLength(ids_arr);
    if (failed(env, ptr(h), deepj_runner_reset(ptr(h)))) return nullptr;
    std::vector<float> logits((size_t)n * (size_t)vocab);
    jint *ids = env->GetIntArrayElements(ids_arr, nullptr);
    int rc = deepj_runner_prefill(ptr(h), reinterpret_cast<const int32_t *>(ids), n, logits.data(), 0);
    env->ReleaseIntArrayElements(ids_arr, ids, JNI_ABORT);
    if (failed(env, ptr(h), rc)) return nullptr;
    jfloatArray out = env->NewFloatArray((jsize)logits.size());
    if (out != nullptr) env->SetFloatArrayRegion(out, 0, (jsize)logits.size(), logits.data());
    return out;
}

JNIEXPORT jintArray JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipRunnerNative_generate(
    JNIEnv *env, jclass, jlong h, jintArray prompt_arr, jint max_new, jfloat temperature, jint top_k, jlong seed,
    jint mode) {
    jint n = env->GetArrayLength(prompt_arr);
    std::vector<int32_t> out((size_t)n + (size_t)(max_new > 0 ? max_new : 0));
    jint *prompt = env->GetIntArrayElements(prompt_arr, nullptr);
    int rc = deepj_runner_generate(ptr(h), reinterpret_cast<const int32_t *>(prompt), n, max_new, temperature, top_k,
                                   seed, mode, out.data());
    env->ReleaseIntArrayElements(prompt_arr, prompt, JNI_ABORT);
    if (failed(env, ptr(h), rc)) return nullptr;
    jintArray res = env->NewIntArray((jsize)out.size());
    if (res != nullptr) env->SetIntArrayRegion(res, 0, (jsize)out.size(), reinterpret_cast<const jint *>(out.data()));
    return res;
}

}  // extern "C"
