// JNI shim: the five native methods of io.github.kirstenali.deepj.tensor.hip.HipNative, each a
// one-to-one wrapper over the C ABI in include/deepj_hip.h.  It takes the place of the JNI
// entry points of the reference's Metal library (native/deepj_metal_jni.mm:1480-1556):
// same signatures, same array handling - inputs released with JNI_ABORT, the download target
// with mode 0 - and native failures surface as java.lang.RuntimeException
// (deepj_metal_jni.mm:888-893).
//
// Build (needs a JDK for jni.h; not part of the default build because the build image has none):
//   hipcc -shared -fPIC -I$JAVA_HOME/include -I$JAVA_HOME/include/linux \
//         deepj_hip_jni.cpp -L.. -ldeepj_hip -o libdeepj_hip_jni.so
#include <jni.h>

#include "../../include/deepj_hip.h"

namespace {

void throw_runtime(JNIEnv *env, const char *msg) {
    jclass cls = env->FindClass("java/lang/RuntimeException");
    if (cls != nullptr) env->ThrowNew(cls, msg);
}

inline void check(JNIEnv *env, int rc) {
    if (rc != 0) throw_runtime(env, deepj_hip_last_error());
}

}  // namespace

extern "C" {

JNIEXPORT void JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipNative_nativeAllocBuffers(
    JNIEnv *env, jclass, jintArray ids_arr, jintArray sizes_arr, jint count) {
    jint *ids = env->GetIntArrayElements(ids_arr, nullptr);
    jint *sizes = env->GetIntArrayElements(sizes_arr, nullptr);
    int rc = deepj_hip_alloc_buffers(reinterpret_cast<const int32_t *>(ids), reinterpret_cast<const int32_t *>(sizes), count);
    env->ReleaseIntArrayElements(ids_arr, ids, JNI_ABORT);
    env->ReleaseIntArrayElements(sizes_arr, sizes, JNI_ABORT);
    check(env, rc);
}

JNIEXPORT void JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipNative_nativeUploadBuffer(
    JNIEnv *env, jclass, jint buf_id, jfloatArray data_arr) {
    jint len = env->GetArrayLength(data_arr);            // the array length, not the allocated size
    jfloat *data = env->GetFloatArrayElements(data_arr, nullptr);
    int rc = deepj_hip_upload(buf_id, data, len);
    env->ReleaseFloatArrayElements(data_arr, data, JNI_ABORT);
    check(env, rc);
}

JNIEXPORT void JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipNative_nativeDownloadBuffer(
    JNIEnv *env, jclass, jint buf_id, jfloatArray out_arr) {
    jint len = env->GetArrayLength(out_arr);
    jfloat *out = env->GetFloatArrayElements(out_arr, nullptr);
    int rc = deepj_hip_download(buf_id, out, len);
    env->ReleaseFloatArrayElements(out_arr, out, 0);     // copy back
    check(env, rc);
}

JNIEXPORT void JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipNative_nativeReleaseBuffers(
    JNIEnv *env, jclass, jintArray ids_arr, jint count) {
    jint *ids = env->GetIntArrayElements(ids_arr, nullptr);
    int rc = deepj_hip_release(reinterpret_cast<const int32_t *>(ids), count);
    env->ReleaseIntArrayElements(ids_arr, ids, JNI_ABORT);
    check(env, rc);
}

JNIEXPORT void JNICALL Java_io_github_kirstenali_deepj_tensor_hip_HipNative_nativeFlushOps(
    JNIEnv *env, jclass, jintArray cmd_arr, jint cmd_len) {
    jint *cmd = env->GetIntArrayElements(cmd_arr, nullptr);
    int rc = deepj_hip_flush_ops(reinterpret_cast<const int32_t *>(cmd), cmd_len);
    env->ReleaseIntArrayElements(cmd_arr, cmd, JNI_ABORT);
    check(env, rc);
}

}  // extern "C"
