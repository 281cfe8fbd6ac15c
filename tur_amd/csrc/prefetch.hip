// turq_weight_prefetch: a read-only pass over a weight's bytes on a stream of its own, so that the memory system works on the
// NEXT launch's weights while the current launch starts, runs and drains.  A decode launch of a few tens of MB spends a third of
// its time before its first bytes arrive and after its last request has left (whatever the kernel does), and a launch cannot
// start before the one that produces its activations has ended - but its weights depend on nothing.  Bytes that have been read
// once sit in the memory-side cache (256 MB on an MI355X) when the matmul asks for them.
#include <hip/hip_ext.h>

#include "mfma_common.h"

namespace {

// every wave keeps D chunks of 4 KiB in flight (D * 4 loads of 16 bytes per lane) and only xors what arrives
template <int D>
__global__ void __launch_bounds__(256) prefetch_kernel(const uint8_t *__restrict__ buf, size_t nchunks, uint32_t *__restrict__ sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const size_t stride = (size_t)gridDim.x * nw;
    size_t c = (size_t)blockIdx.x * nw + wave;
    uint4v r[D][4];
    uint4v acc = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int d = 0; d < D; d++) {
        const size_t cc = c + d * stride;
        const uint8_t *p = buf + (cc < nchunks ? cc : 0) * 4096 + 16 * lane;
#pragma unroll
        for (int i = 0; i < 4; i++) r[d][i] = *(const uint4v *)(p + 1024 * i);
    }
    while (c < nchunks) {
#pragma unroll
        for (int d = 0; d < D; d++) {
#pragma unroll
            for (int i = 0; i < 4; i++) acc ^= r[d][i];
            const size_t cn = c + D * stride;
            const uint8_t *p = buf + (cn < nchunks ? cn : 0) * 4096 + 16 * lane;
#pragma unroll
            for (int i = 0; i < 4; i++) r[d][i] = *(const uint4v *)(p + 1024 * i);
            c += stride;
        }
    }
    // never true for memory that holds anything but this one pattern: the loads must not be optimised away
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u && sink) sink[blockIdx.x] = acc.x;
}

}  // namespace

// reads the first nbytes / 4096 * 4096 bytes at buf (16-byte aligned) with `workgroups` four-wave workgroups
hipError_t turq_launch_weight_prefetch(const void *buf, size_t nbytes, int workgroups, int depth, hipStream_t stream, hipEvent_t ev_start,
                                       hipEvent_t ev_stop) {
    if (workgroups < 1 || ((uintptr_t)buf & 15) != 0) return hipErrorInvalidValue;
    const size_t nchunks = nbytes / 4096;
    if (nchunks == 0) return hipSuccess;
    const size_t most = (nchunks + 3) / 4;  // no more workgroups than there are chunks for
    if ((size_t)workgroups > most) workgroups = (int)most;
    auto kern = depth >= 4 ? prefetch_kernel<4> : depth >= 2 ? prefetch_kernel<2> : prefetch_kernel<1>;
    if (ev_start) {
        hipExtLaunchKernelGGL(kern, dim3((unsigned)workgroups), dim3(256), 0, stream, ev_start, ev_stop, 0, (const uint8_t *)buf, nchunks,
                              (uint32_t *)nullptr);
        return hipGetLastError();
    }
    kern<<<dim3((unsigned)workgroups), dim3(256), 0, stream>>>((const uint8_t *)buf, nchunks, (uint32_t *)nullptr);
    return hipGetLastError();
}
