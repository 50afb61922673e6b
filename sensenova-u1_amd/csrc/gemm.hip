// LDS-staged dequant-GEMM on bf16 MFMA (M > 16), with modality-grouped row routing.
//
// y[m][n] = sum_k x[m][k] * w[n][k].  A workgroup of four wavefronts owns a BM x BN output
// tile and walks K in steps of BK = 64: the activation tile is copied to LDS as is, the packed
// weight tile is decoded to bf16 (with the rounding chain the numerics mode asks for) and
// written to LDS, then each wavefront runs v_mfma_f32_32x32x16_bf16 over its 64 x 64 quadrant
// with the weight rows as the A operand and the activation rows as the B operand, so that a
// lane ends up with runs of four consecutive output columns of one activation row.
//
// Row routing: the M rows are seen through an optional row map as [group 0 | group 1]; group 0
// multiplies the first weight set (text rows -> understanding weights), group 1 the second
// (image rows -> generation weights).  blockIdx.y enumerates the row tiles of group 0, then
// those of group 1; a plain linear is the case "all rows in group 0, no map".

#include "sngguf_common.hpp"
#include "gemm_args.hpp"

namespace sngguf {

constexpr int BM = 128;      // activation rows per tile
constexpr int BN = 128;      // weight rows (output columns) per tile
constexpr int BK = 64;       // K step
constexpr int LDS_LD = 72;   // bf16 elements per LDS row: 144 bytes, keeps 16-byte reads conflict-free


template <int QT, int NUM>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs a) {
    __shared__ __attribute__((aligned(16))) bf16_t xs[BM * LDS_LD];
    __shared__ __attribute__((aligned(16))) bf16_t ws[BN * LDS_LD];

    const int tid = threadIdx.x, lane = tid & 63;
    // the wavefront index is the same in all lanes: holding it in a scalar register keeps every address derived
    // from it (LDS slabs, tile rows) in scalar arithmetic
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- which rows does this tile cover --------------------------------------------------
    const int64_t n0 = a.n0_dev ? (int64_t)*a.n0_dev : a.n0;
    const int64_t t0 = (n0 + BM - 1) / BM, t1 = (a.M - n0 + BM - 1) / BM;
    const int64_t ty = blockIdx.y;
    int g;
    int64_t row_begin, row_end;
    if (ty < t0) {
        g = 0; row_begin = ty * BM; row_end = n0;
    } else if (ty < t0 + t1) {
        g = 1; row_begin = n0 + (ty - t0) * BM; row_end = a.M;
    } else {
        return;
    }
    if (!((a.group_mask >> g) & 1)) return;
    if (row_end > row_begin + BM) row_end = row_begin + BM;
    const uint8_t* __restrict__ q = a.q[g];
    const bf16_t* __restrict__ bias = a.bias[g];
    const int64_t nb0 = (int64_t)blockIdx.x * BN;
    const int64_t row_bytes = a.K / Fmt<QT>::bs * Fmt<QT>::ts;

    // ---- per-thread load assignments ---------------------------------------------------------
    // activations: 128 rows x 8 chunks of 16 bytes, four chunks per thread
    const bf16_t* xsrc[4];
    int xdst[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int f = tid + 256 * i, r = f >> 3, c = f & 7;
        const int64_t rr = row_begin + r;
        xdst[i] = r * LDS_LD + 8 * c;
        if (rr < row_end) {
            const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
            xsrc[i] = a.x + gr * a.K + 8 * c;
        } else {
            xsrc[i] = nullptr;
        }
    }
    // weights: 128 rows x 64 elements, 32 consecutive elements per thread
    const int wr = tid >> 1, wh = tid & 1;
    int64_t wrow = nb0 + wr;
    if (wrow >= a.N) wrow = a.N - 1;
    const uint8_t* __restrict__ wsrc = q + wrow * row_bytes;
    const int wdst = wr * LDS_LD + 32 * wh;

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    const int64_t ksteps = (a.K + BK - 1) / BK;
    for (int64_t kb = 0; kb < ksteps; kb++) {
        const int64_t k0 = kb * BK;
        // -- global -> registers
        u32x4_t xv[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // K is a multiple of 32, so a 64-wide step can run 32 elements past the end (Q8_0 only)
            const bool ok = xsrc[i] != nullptr && (k0 + 8 * ((tid + 256 * i) & 7) < a.K);
            xv[i] = ok ? *reinterpret_cast<const u32x4_t*>(xsrc[i] + k0) : u32x4_t{0u, 0u, 0u, 0u};
        }
        u32x4_t wv[4];
        if (k0 + 32 * wh < a.K) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float w[8];
                decode8<QT, NUM>(wsrc, k0 + 32 * wh + 8 * j, w);
#pragma unroll
                for (int p = 0; p < 4; p++) wv[j][p] = pack_bf16(w[2 * p], w[2 * p + 1]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) wv[j] = u32x4_t{0u, 0u, 0u, 0u};
        }
        __syncthreads();  // the previous step's MFMA reads are done
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<u32x4_t*>(&xs[xdst[i]]) = xv[i];
#pragma unroll
        for (int j = 0; j < 4; j++) *reinterpret_cast<u32x4_t*>(&ws[wdst + 8 * j]) = wv[j];
        __syncthreads();
        // -- MFMA over the four 16-wide K slices
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const int kk = ks * 16 + 8 * (lane >> 5);
            bf16x8_t af[2], bfr[2];
#pragma unroll
            for (int i = 0; i < 2; i++)
                af[i] = *reinterpret_cast<const bf16x8_t*>(&ws[(wn * 64 + i * 32 + (lane & 31)) * LDS_LD + kk]);
#pragma unroll
            for (int j = 0; j < 2; j++)
                bfr[j] = *reinterpret_cast<const bf16x8_t*>(&xs[(wm * 64 + j * 32 + (lane & 31)) * LDS_LD + kk]);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
    }

    // ---- epilogue: D[i][j], i = weight row (n), j = activation row (m) ------------------------------
    // lane: j = lane % 32; register v: i = 8 * (v / 4) + 4 * (lane / 32) + v % 4
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int64_t rr = row_begin + wm * 64 + j * 32 + (lane & 31);
        if (rr >= row_end) continue;
        const int64_t gr = a.rowmap ? (int64_t)a.rowmap[rr] : rr;
        bf16_t* yrow = a.y + gr * a.N;
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int vg = 0; vg < 4; vg++) {
                const int64_t n = nb0 + wn * 64 + i * 32 + 8 * vg + 4 * (lane >> 5);
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float b = (bias && n + e < a.N) ? bf16_to_f32(bias[n + e]) : 0.f;
                    o[e] = n + e < a.N ? add_residual(acc[i][j][4 * vg + e] + b, a.residual, gr * a.N + n + e) : 0.f;
                }
                if (n + 3 < a.N && (a.N & 3) == 0) {
                    u32x2_t pk = {pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3])};
                    *reinterpret_cast<u32x2_t*>(yrow + n) = pk;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < a.N) yrow[n + e] = f32_to_bf16(o[e]);
                }
            }
        }
    }
}

// ---- row partition for the indicator form of the grouped launcher ---------------------------------
// One workgroup: stable partition of row indices by indicator == 0 / != 0.
// workspace layout: int32 n0 at [0], padding to 16 bytes, then M int32 row indices.
__global__ __launch_bounds__(1024) void partition_rows_kernel(const uint8_t* __restrict__ indicator, int64_t M,
                                                              int32_t* __restrict__ ws) {
    __shared__ int32_t zeros_before[1024];
    __shared__ int32_t ones_before[1024];
    const int tid = threadIdx.x;
    const int64_t per = (M + 1023) / 1024;
    const int64_t b = tid * per, e = (b + per < M) ? b + per : M;
    int32_t z = 0, o = 0;
    for (int64_t i = b; i < e; i++) {
        if (indicator[i]) o++; else z++;
    }
    zeros_before[tid] = z;
    ones_before[tid] = o;
    __syncthreads();
    // inclusive Hillis-Steele scan over the 1024 per-thread counts
    for (int off = 1; off < 1024; off <<= 1) {
        int32_t zv = 0, ov = 0;
        if (tid >= off) { zv = zeros_before[tid - off]; ov = ones_before[tid - off]; }
        __syncthreads();
        zeros_before[tid] += zv;
        ones_before[tid] += ov;
        __syncthreads();
    }
    const int32_t total_zero = zeros_before[1023];
    int32_t zpos = zeros_before[tid] - z;
    int32_t opos = total_zero + ones_before[tid] - o;
    int32_t* map = ws + 4;
    for (int64_t i = b; i < e; i++) {
        if (indicator[i]) map[opos++] = (int32_t)i; else map[zpos++] = (int32_t)i;
    }
    if (tid == 0) ws[0] = total_zero;
}

// ---- host-side dispatch ---------------------------------------------------------------------------------

template <int QT>
static int launch_num(const GemmArgs& a, int numerics, hipStream_t stream) {
    const int64_t row_tiles = (a.M + BM - 1) / BM + 1;  // a split adds at most one partial tile
    dim3 grid((unsigned)((a.N + BN - 1) / BN), (unsigned)row_tiles), block(256);
    if (numerics == SNGGUF_NUM_GGML_FP32) gemm_kernel<QT, SNGGUF_NUM_GGML_FP32><<<grid, block, 0, stream>>>(a);
    else if (numerics == SNGGUF_NUM_UPSTREAM_FP16) gemm_kernel<QT, SNGGUF_NUM_UPSTREAM_FP16><<<grid, block, 0, stream>>>(a);
    else return SNGGUF_E_BADTYPE;
    return hipGetLastError() == hipSuccess ? SNGGUF_OK : SNGGUF_E_LAUNCH;
}

int launch_gemm_tiles(const GemmArgs& a, int qtype, int numerics, hipStream_t stream);

static int launch_type(const GemmArgs& a, int qtype, int numerics, hipStream_t stream) {
    // Q8_0 / Q4_K beyond the decode kernels' 64 rows: the large-tile kernel, also where its 256 x 256 tiles are few
    // or mostly empty (measured at 65 ... 1024 rows on the four projection shapes of the 8B model: 10 - 25 % faster
    // than the 128 x 128 kernel below, whose K loop is the slower one per step); everything else: the 128 x 128 kernel
    if (qtype == 30) return launch_gemm_tiles(a, 30, numerics, stream);  // weights already bf16 (workspace routes)
    const bool tile_type = (qtype == SNGGUF_TYPE_Q8_0 && a.K % 64 == 0) || qtype == SNGGUF_TYPE_Q4_K;
    // (the large-tile kernel addresses activations with 32-bit byte offsets)
    const bool x_fits = a.M * a.K < ((int64_t)1 << 31);
    if (tile_type && x_fits && a.M >= 65) return launch_gemm_tiles(a, qtype, numerics, stream);
#define SNGGUF_CALL(QT) launch_num<QT>(a, numerics, stream)
    SNGGUF_DISPATCH_TYPE(qtype, SNGGUF_CALL)
#undef SNGGUF_CALL
}

int launch_gemm(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias,
                const void* residual, void* y,
                int numerics, hipStream_t stream) {
    GemmArgs a{};
    a.x = static_cast<const bf16_t*>(x);
    a.y = static_cast<bf16_t*>(y);
    a.M = M; a.N = N; a.K = K;
    a.rowmap = nullptr; a.n0_dev = nullptr; a.n0 = M;
    a.q[0] = a.q[1] = static_cast<const uint8_t*>(q);
    a.bias[0] = a.bias[1] = static_cast<const bf16_t*>(bias);
    a.residual = static_cast<const bf16_t*>(residual);
    a.group_mask = 1;
    return launch_type(a, qtype, numerics, stream);
}

// y = x w^T (+ bias) with w already bf16 [N][K]: the tile kernel without its decode stage.
// Needs K % 64 == 0 and M K < 2^31 (checked by the caller).
int launch_gemm_dense(const void* x, int64_t M, const void* w, int64_t N, int64_t K, const void* bias, void* y,
                      hipStream_t stream) {
    GemmArgs a{};
    a.x = static_cast<const bf16_t*>(x);
    a.y = static_cast<bf16_t*>(y);
    a.M = M; a.N = N; a.K = K;
    a.rowmap = nullptr; a.n0_dev = nullptr; a.n0 = M;
    a.q[0] = a.q[1] = static_cast<const uint8_t*>(w);
    a.bias[0] = a.bias[1] = static_cast<const bf16_t*>(bias);
    a.residual = nullptr;
    a.group_mask = 1;
    return launch_gemm_tiles(a, 30, SNGGUF_NUM_GGML_FP32, stream);
}

int launch_gemm_dense4(const GemmArgs& a, hipStream_t stream);

// h = silu(x wg^T) * (x wu^T) with both weights already bf16 and interleaved in blocks of 128 rows (w2: rows2 =
// 256 ceil(cols / 128) rows of K, as launch_dequantize_interleaved writes them): one launch of the four-wavefront dense
// kernel with the gated epilogue.  Needs K % 128 == 0 (an even number of K steps), cols % 8 == 0 and M K < 2^31
// (checked by the caller).
int launch_gemm_dense_gated(const void* x, int64_t M, const void* w2, int64_t cols, int64_t K, void* h, hipStream_t stream) {
    GemmArgs a{};
    a.x = static_cast<const bf16_t*>(x);
    a.y = static_cast<bf16_t*>(h);
    a.M = M; a.N = 256 * ((cols + 127) / 128); a.K = K;
    a.rowmap = nullptr; a.n0_dev = nullptr; a.n0 = M;
    a.q[0] = a.q[1] = static_cast<const uint8_t*>(w2);
    a.group_mask = 1;
    a.gated_cols = cols;
    return launch_gemm_dense4(a, stream);
}

int launch_splitk_reduce(const GemmArgs& a, const uint8_t* indicator, int64_t n_text, hipStream_t stream);

// y = x W^T (+ bias) on the large-tile kernel with K split over `slices` workgroups per output tile: fp32 partial
// sums into `partial` (slices * M * N floats), then one pass that adds them.  For problems whose tiles alone leave
// most of the chip idle.  qtype: Q8_0 (K % 64 == 0), Q4_K, or 30 for weights that are already bf16; 2 <= slices <=
// K / 64; M K < 2^31 (checked by the caller).
int launch_gemm_splitk(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias, void* y,
                       float* partial, int slices, int numerics, hipStream_t stream) {
    GemmArgs a{};
    a.x = static_cast<const bf16_t*>(x);
    a.y = static_cast<bf16_t*>(y);
    a.M = M; a.N = N; a.K = K;
    a.rowmap = nullptr; a.n0_dev = nullptr; a.n0 = M;
    a.q[0] = a.q[1] = static_cast<const uint8_t*>(q);
    a.bias[0] = a.bias[1] = static_cast<const bf16_t*>(bias);
    a.residual = nullptr;
    a.group_mask = 1;
    a.partial = partial;
    a.ksplit = slices;
    const int rc = launch_gemm_tiles(a, qtype, qtype == 30 ? SNGGUF_NUM_GGML_FP32 : numerics, stream);
    if (rc != SNGGUF_OK) return rc;
    return launch_splitk_reduce(a, nullptr, M, stream);
}

int64_t grouped_workspace_bytes(int64_t M) { return 16 + 4 * (M > 0 ? M : 0); }

int launch_grouped_gemm(const void* x, int64_t M, const uint8_t* indicator, int64_t n_text, const void* q_und,
                        int qtype_und, const void* q_gen, int qtype_gen, int64_t N, int64_t K, const void* bias_und,
                        const void* bias_gen, void* y, void* workspace, int numerics, hipStream_t stream, float* partial,
                        int slices) {
    // partial / slices: K split over `slices` workgroups per tile with fp32 partial sums (slices * M * N floats);
    // only for two weight sets of one type that the large-tile kernel takes (checked by the caller)
    GemmArgs a{};
    a.x = static_cast<const bf16_t*>(x);
    a.y = static_cast<bf16_t*>(y);
    a.M = M; a.N = N; a.K = K;
    a.q[0] = static_cast<const uint8_t*>(q_und);
    a.q[1] = static_cast<const uint8_t*>(q_gen);
    a.bias[0] = static_cast<const bf16_t*>(bias_und);
    a.bias[1] = static_cast<const bf16_t*>(bias_gen);
    a.residual = nullptr;
    if (indicator) {
        int32_t* ws = static_cast<int32_t*>(workspace);
        partition_rows_kernel<<<1, 1024, 0, stream>>>(indicator, M, ws);
        if (hipGetLastError() != hipSuccess) return SNGGUF_E_LAUNCH;
        a.rowmap = ws + 4;
        a.n0_dev = ws;
        a.n0 = 0;
    } else {
        a.rowmap = nullptr;
        a.n0_dev = nullptr;
        a.n0 = n_text;
    }
    if (partial && slices > 1) {
        if (qtype_und != qtype_gen) return SNGGUF_E_BADTYPE;
        a.group_mask = 3;
        a.partial = partial;
        a.ksplit = slices;
        const int rc = launch_gemm_tiles(a, qtype_und, numerics, stream);
        if (rc != SNGGUF_OK) return rc;
        return launch_splitk_reduce(a, indicator, n_text, stream);
    }
    if (qtype_und == qtype_gen) {
        a.group_mask = 3;
        return launch_type(a, qtype_und, numerics, stream);
    }
    a.group_mask = 1;
    int rc = launch_type(a, qtype_und, numerics, stream);
    if (rc != SNGGUF_OK) return rc;
    a.group_mask = 2;
    return launch_type(a, qtype_gen, numerics, stream);
}

}  // namespace sngguf
