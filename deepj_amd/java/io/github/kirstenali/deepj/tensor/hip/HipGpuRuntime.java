package io.github.kirstenali.deepj.tensor.hip;

import io.github.kirstenali.deepj.tensor.GpuRuntime;

/** {@link GpuRuntime} over the HIP native library: five pass-throughs. */
public final class HipGpuRuntime implements GpuRuntime {

    public HipGpuRuntime() {
        if (!HipNative.AVAILABLE) {
            throw new IllegalStateException("DeepJ HIP native library is not available on this machine");
        }
    }

    @Override
    public void allocBuffers(int[] ids, int[] sizes, int count) {
        HipNative.nativeAllocBuffers(ids, sizes, count);
    }

    @Override
    public void uploadBuffer(int bufId, float[] data) {
        HipNative.nativeUploadBuffer(bufId, data);
    }

    @Override
    public void downloadBuffer(int bufId, float[] out) {
        HipNative.nativeDownloadBuffer(bufId, out);
    }

    @Override
    public void releaseBuffers(int[] ids, int count) {
        HipNative.nativeReleaseBuffers(ids, count);
    }

    @Override
    public void flushOps(int[] cmdStream, int cmdStreamLength) {
        HipNative.nativeFlushOps(cmdStream, cmdStreamLength);
    }
}
