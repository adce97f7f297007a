// Calibration kernels for the benchmark's roofline lines (no counterpart in the reference): what a kernel that only
// reads a buffer reaches on this part, and what one that only issues int8 matrix instructions reaches.  They measure
// the machine, not the library: the peaks in the roofline fractions stay the published ones.
#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kReadUnroll = 8;  // 16-byte loads in flight per lane

// Grid-stride read of n16 16-byte pieces, kReadUnroll loads in flight per lane; the xor keeps the loads alive.
template <bool kNonTemporal>
__global__ void __launch_bounds__(256) read_stream_kernel(const u32x4 *__restrict__ p, size_t n16, uint32_t *__restrict__ sink) {
    const size_t tid = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    uint32_t acc = 0;
    size_t i = tid;
    for (; i + (kReadUnroll - 1) * stride < n16; i += kReadUnroll * stride) {
        u32x4 v[kReadUnroll];
#pragma unroll
        for (int u = 0; u < kReadUnroll; u++) v[u] = kNonTemporal ? __builtin_nontemporal_load(&p[i + u * stride]) : p[i + u * stride];
#pragma unroll
        for (int u = 0; u < kReadUnroll; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) {
        const u32x4 v = kNonTemporal ? __builtin_nontemporal_load(&p[i]) : p[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u) sink[tid & 255] = acc;  // practically never: the result is not wanted
}

// Four independent accumulator chains of v_mfma_i32_32x32x32_i8 per wave, operands in registers, nothing else.
__global__ void __launch_bounds__(512) mfma_i8_kernel(int *__restrict__ sink, uint32_t iters) {
    const int lane = threadIdx.x & 63;
    const v4i a = {lane, lane * 3 + 1, 0x01020304, 0x7f807f80}, b = {lane ^ 21, 0x11111111, lane * 5, 0x0f0f0f0f};
    v16i c0 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
    for (uint32_t i = 0; i < iters; i++) {
        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, a, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, a, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, b, c3, 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int r = 0; r < 16; r++) s += c0[r] ^ c1[r] ^ c2[r] ^ c3[r];
    if (s == 0x12345678) sink[threadIdx.x & 255] = s;
}

}  // namespace

void launch_calib_read(const void *dev, size_t bytes, bool non_temporal, uint32_t *sink, hipStream_t stream) {
    const size_t n16 = bytes / 16;
    if (n16 == 0) return;
    // 2048 workgroups of 256 lanes with 8 loads each hold 64 MB in flight: measured best for 33 MB ... 431 MB
    const dim3 grid(bytes >= (size_t(200) << 20) ? 16384 : 2048), block(256);
    if (non_temporal)
        hipLaunchKernelGGL(read_stream_kernel<true>, grid, block, 0, stream, static_cast<const u32x4 *>(dev), n16, sink);
    else
        hipLaunchKernelGGL(read_stream_kernel<false>, grid, block, 0, stream, static_cast<const u32x4 *>(dev), n16, sink);
}

uint64_t launch_calib_mfma_i8(uint32_t iters, uint32_t workgroups, int *sink, hipStream_t stream) {
    if (iters == 0 || workgroups == 0) return 0;
    hipLaunchKernelGGL(mfma_i8_kernel, dim3(workgroups), dim3(512), 0, stream, sink, iters);
    // ops: 8 waves x 4 chains x iters instructions of 32 x 32 x 32 multiply-adds (2 ops each)
    return static_cast<uint64_t>(workgroups) * 8 * 4 * iters * 65536ull;
}

}  // namespace rnb
