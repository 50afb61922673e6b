// A plain streaming read of device memory, for measurement only: what rate this device's memory system gives a
// launch that does nothing but read every byte once.  Each workgroup walks its own contiguous share of the buffer in
// 16-byte pieces per lane (a wavefront request covers 1 KB = eight whole 128-byte lines), eight requests in flight per
// lane, with the non-temporal hint the decode kernels use for weights that are read once; the values are folded into
// one word per workgroup so that no load can be dropped.  The bench reports the rate next to the published peak: it is
// the ceiling a decode kernel of the same size can be compared with.
#include "sngguf_common.hpp"

namespace sngguf {

namespace {
constexpr int kProbeThreads = 512;
constexpr int kProbeUnroll = 8;
}  // namespace

template <bool NT>
__global__ __launch_bounds__(kProbeThreads) void stream_read_kernel(const u32x4_t* __restrict__ p, int64_t pieces, uint32_t* __restrict__ out) {
    // workgroup b reads pieces [b * share, (b + 1) * share): contiguous, so that consecutive requests of a compute
    // unit stay in one DRAM page as long as possible
    const int64_t share = (pieces + gridDim.x - 1) / gridDim.x;
    const int64_t lo = (int64_t)blockIdx.x * share;
    const int64_t hi = lo + share < pieces ? lo + share : pieces;
    uint32_t acc = 0;
    int64_t i = lo + threadIdx.x;
    for (; i + (int64_t)(kProbeUnroll - 1) * kProbeThreads < hi; i += (int64_t)kProbeUnroll * kProbeThreads) {
        u32x4_t v[kProbeUnroll];
#pragma unroll
        for (int u = 0; u < kProbeUnroll; u++) v[u] = NT ? __builtin_nontemporal_load(p + i + (int64_t)u * kProbeThreads) : p[i + (int64_t)u * kProbeThreads];
#pragma unroll
        for (int u = 0; u < kProbeUnroll; u++) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
    for (; i < hi; i += kProbeThreads) {
        const u32x4_t v = NT ? __builtin_nontemporal_load(p + i) : p[i];
        acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) acc ^= (uint32_t)__shfl_xor((int)acc, s, 64);
    __shared__ uint32_t part[kProbeThreads / 64];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
#pragma unroll
        for (int w = 0; w < kProbeThreads / 64; w++) t ^= part[w];
        out[blockIdx.x] = t;
    }
}

int64_t stream_probe_out_bytes() { return 4 * 4096; }

// `workgroups` <= 4096; 0 picks one per compute unit times four (1024 on a 256-unit device).
int launch_stream_read(const void* p, int64_t bytes, void* out, int workgroups, bool nontemporal, hipStream_t stream) {
    const int64_t pieces = bytes / 16;
    if (pieces == 0) return SNGGUF_OK;
    int wg = workgroups > 0 ? workgroups : 1024;
    if (wg > 4096) wg = 4096;
    if (nontemporal)
        stream_read_kernel<true><<<dim3((unsigned)wg), dim3(kProbeThreads), 0, stream>>>(static_cast<const u32x4_t*>(p), pieces, static_cast<uint32_t*>(out));
    else
        stream_read_kernel<false><<<dim3((unsigned)wg), dim3(kProbeThreads), 0, stream>>>(static_cast<const u32x4_t*>(p), pieces, static_cast<uint32_t*>(out));
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

}  // namespace sngguf
