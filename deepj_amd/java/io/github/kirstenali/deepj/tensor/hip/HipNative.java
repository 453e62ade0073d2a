package io.github.kirstenali.deepj.tensor.hip;

import java.io.InputStream;
import java.nio.file.Files;
import java.nio.file.Path;
import java.nio.file.StandardCopyOption;

/**
 * JNI bridge to the MI355X runtime (libdeepj_hip_jni.so, which links libdeepj_hip.so).
 * Five calls, one per {@link io.github.kirstenali.deepj.tensor.GpuRuntime} method.
 */
final class HipNative {

    static final boolean AVAILABLE;

    static {
        boolean loaded = false;
        try {
            loadFromResources("/native/linux/libdeepj_hip.so");
            loadFromResources("/native/linux/libdeepj_hip_jni.so");
            loaded = true;
        } catch (Throwable t) {
            System.err.println("[DeepJ/HIP] Failed to load native library: " + t);
        }
        AVAILABLE = loaded;
    }

    private HipNative() {}

    private static void loadFromResources(String resource) throws Exception {
        try (InputStream in = HipNative.class.getResourceAsStream(resource)) {
            if (in == null) throw new IllegalStateException("missing resource " + resource);
            String name = resource.substring(resource.lastIndexOf('/') + 1);
            Path dir = Files.createTempDirectory("deepj-hip");
            Path tmp = dir.resolve(name);
            Files.copy(in, tmp, StandardCopyOption.REPLACE_EXISTING);
            tmp.toFile().deleteOnExit();
            dir.toFile().deleteOnExit();
            System.load(tmp.toAbsolutePath().toString());
        }
    }

    static native void nativeAllocBuffers(int[] ids, int[] sizes, int count);

    static native void nativeUploadBuffer(int bufId, float[] data);

    static native void nativeDownloadBuffer(int bufId, float[] out);

    static native void nativeReleaseBuffers(int[] ids, int count);

    static native void nativeFlushOps(int[] cmdStream, int cmdStreamLength);
}
