// extern "C" entry points of libsngguf: argument validation and routing to the kernel
// launchers.  Nothing here allocates, synchronises or throws.
#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include "../../include/sngguf.h"

namespace sngguf {
int launch_dequantize(const void* q, int qtype, int64_t rows, int64_t cols, void* out, int out_dtype, int numerics,
                      hipStream_t stream);
int launch_gemv(const void* x, int64_t M, const void* qa, const void* qb, int qtype, int64_t N, int64_t K,
                const void* bias, const void* residual, void* y, int numerics, bool gated, hipStream_t stream);
int launch_gemv_q8_mfma(const void* x, int64_t M, const void* qa, const void* qb, int64_t N, int64_t K, const void* bias,
                        const void* residual, void* y, int numerics, bool gated, hipStream_t stream, const void* gamma,
                        float eps, uint64_t* amax = nullptr);
int launch_gemv_kq_mfma(const void* x, int64_t M, const void* qa, const void* qb, int qtype, int64_t N, int64_t K,
                        const void* bias, const void* residual, void* y, int numerics, bool gated, hipStream_t stream,
                        const void* gamma, float eps, uint64_t* amax = nullptr);
int64_t gemv_argmax_slots(int qtype, int64_t M, int64_t N);
int launch_argmax_reduce(const uint64_t* keys, int64_t M, int64_t slots, int64_t* out_index, hipStream_t stream);
int launch_dequantize_bf16(const void* q, int64_t rows, int64_t cols, void* out, int out_dtype, hipStream_t stream);
int launch_gemv_bf16(const void* x, int64_t M, const void* wa, const void* wb, int64_t N, int64_t K, const void* bias,
                     const void* residual, void* y, bool gated, hipStream_t stream);
int launch_rmsnorm(const void* x, int64_t M, int64_t K, const void* gamma, float eps, void* y, hipStream_t stream);
int64_t q8_0_tiled_bytes(int64_t N, int64_t K);
int64_t static_scratch_bytes();
int static_scratch(void** ptr);
int launch_q8_0_tile(const void* q, int64_t N, int64_t K, void* tiled, hipStream_t stream);
int launch_gemv_q8_tiled(const void* x, int64_t M, const void* ta, const void* tb, int64_t N, int64_t K, const void* bias,
                         const void* residual, void* y, int numerics, bool gated, hipStream_t stream,
                         const void* gamma = nullptr, float eps = 0.f);
int launch_gemm_splitk(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias, void* y,
                       float* partial, int slices, int numerics, hipStream_t stream);
int launch_gemm_dense(const void* x, int64_t M, const void* w, int64_t N, int64_t K, const void* bias, void* y,
                      hipStream_t stream);
int launch_dequantize_interleaved(const void* q, int qtype, int64_t rows, int64_t cols, void* out, int second, int numerics,
                                  hipStream_t stream);
int launch_gemm_dense_gated(const void* x, int64_t M, const void* w2, int64_t cols, int64_t K, void* h, hipStream_t stream);
int launch_gemm(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias,
                const void* residual, void* y,
                int numerics, hipStream_t stream);
int64_t mlp_q8_decode_workspace_bytes(int64_t M, int64_t inter);
int64_t mlp_q8_decode_status_offset();
int64_t mlp_q8_decode_ctl_bytes();
bool mlp_q8_decode_fits(int64_t M, int64_t hidden, int64_t inter);
int launch_mlp_q8_decode(const void* x, int64_t M, const void* gamma, float eps, const void* q_gate, const void* q_up, const void* q_down,
                         int64_t hidden, int64_t inter, const void* residual, void* y, void* workspace, int numerics, int spin_limit,
                         hipStream_t stream);
bool mlp_kq_decode_fits(int qtype_gate_up, int qtype_down, int64_t M, int64_t hidden, int64_t inter);
int launch_mlp_kq_decode(const void* x, int64_t M, const void* gamma, float eps, const void* q_gate, const void* q_up, const void* q_down,
                         int qtype_down, int64_t hidden, int64_t inter, const void* residual, void* y, void* workspace, int numerics,
                         int spin_limit, hipStream_t stream);
int64_t stream_probe_out_bytes();
int launch_stream_read(const void* p, int64_t bytes, void* out, int workgroups, bool nontemporal, hipStream_t stream);
int64_t grouped_workspace_bytes(int64_t M);
int launch_grouped_gemm(const void* x, int64_t M, const uint8_t* indicator, int64_t n_text, const void* q_und,
                        int qtype_und, const void* q_gen, int qtype_gen, int64_t N, int64_t K, const void* bias_und,
                        const void* bias_gen, void* y, void* workspace, int numerics, hipStream_t stream,
                        float* partial = nullptr, int slices = 0);
}  // namespace sngguf

namespace {

constexpr int64_t kMaxDim = (int64_t)1 << 31;  // kernels index rows / columns with 32-bit tile counters

inline bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
inline bool known_type(int t) { return sngguf_block_size(t) != 0; }
inline bool known_numerics(int n) { return n == SNGGUF_NUM_GGML_FP32 || n == SNGGUF_NUM_UPSTREAM_FP16; }

// Shape / pointer checks shared by the matmul entry points.
int check_matmul(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* y, int numerics) {
    if (!known_type(qtype) || !known_numerics(numerics)) return SNGGUF_E_BADTYPE;
    if (M < 0 || N < 0 || K <= 0 || M >= kMaxDim || N >= kMaxDim || K >= kMaxDim) return SNGGUF_E_BADSHAPE;
    if (K % sngguf_block_size(qtype) != 0) return SNGGUF_E_BADSHAPE;
    if (M == 0 || N == 0) return SNGGUF_OK;
    if (!x || !q || !y) return SNGGUF_E_NULLPTR;
    if (!aligned(x, 16) || !aligned(y, 16) || !aligned(q, 16)) return SNGGUF_E_ALIGN;
    return SNGGUF_OK;
}

}  // namespace

extern "C" {

int sngguf_version(void) { return 100; }

const char* sngguf_strerror(int code) {
    switch (code) {
    case SNGGUF_OK: return "ok";
    case SNGGUF_E_BADTYPE: return "unsupported quant type, output dtype or numerics mode";
    case SNGGUF_E_BADSHAPE: return "bad shape (negative, not a multiple of the block size, or too large)";
    case SNGGUF_E_NULLPTR: return "required pointer is NULL";
    case SNGGUF_E_ALIGN: return "pointer is not aligned as required";
    case SNGGUF_E_LAUNCH: return "HIP kernel launch failed";
    case SNGGUF_E_NODEVICE: return "no usable gfx950 device";
    case SNGGUF_E_IO: return "file could not be opened or mapped";
    case SNGGUF_E_FORMAT: return "not a GGUF file, or truncated / corrupt";
    case SNGGUF_E_TOOLARGE: return "problem exceeds the static scratch area of the allocation-free entry point (use sngguf_linear_ws with a caller workspace)";
    default: return "unknown error";
    }
}

int64_t sngguf_type_size(int qtype) {
    switch (qtype) {
    case SNGGUF_TYPE_Q4_0: return 18;
    case SNGGUF_TYPE_Q4_1: return 20;
    case SNGGUF_TYPE_Q5_0: return 22;
    case SNGGUF_TYPE_Q5_1: return 24;
    case SNGGUF_TYPE_Q8_0: return 34;
    case SNGGUF_TYPE_Q2_K: return 84;
    case SNGGUF_TYPE_Q3_K: return 110;
    case SNGGUF_TYPE_Q4_K: return 144;
    case SNGGUF_TYPE_Q5_K: return 176;
    case SNGGUF_TYPE_Q6_K: return 210;
    case SNGGUF_TYPE_BF16: return 2;
    default: return 0;
    }
}

int64_t sngguf_block_size(int qtype) {
    switch (qtype) {
    case SNGGUF_TYPE_Q4_0: case SNGGUF_TYPE_Q4_1: case SNGGUF_TYPE_Q5_0: case SNGGUF_TYPE_Q5_1: case SNGGUF_TYPE_Q8_0:
        return 32;
    case SNGGUF_TYPE_Q2_K: case SNGGUF_TYPE_Q3_K: case SNGGUF_TYPE_Q4_K: case SNGGUF_TYPE_Q5_K: case SNGGUF_TYPE_Q6_K:
        return 256;
    case SNGGUF_TYPE_BF16: return 1;
    default: return 0;
    }
}

int sngguf_dequantize(const void* q, int qtype, int64_t rows, int64_t cols, void* out, int out_dtype, int numerics,
                      void* stream) {
    if (!known_type(qtype) || !known_numerics(numerics)) return SNGGUF_E_BADTYPE;
    if (out_dtype != SNGGUF_OUT_F32 && out_dtype != SNGGUF_OUT_F16 && out_dtype != SNGGUF_OUT_BF16) return SNGGUF_E_BADTYPE;
    if (rows < 0 || cols < 0 || rows >= kMaxDim || cols >= kMaxDim) return SNGGUF_E_BADSHAPE;
    if (cols % sngguf_block_size(qtype) != 0) return SNGGUF_E_BADSHAPE;
    if (rows == 0 || cols == 0) return SNGGUF_OK;
    if (!q || !out) return SNGGUF_E_NULLPTR;
    if (!aligned(q, 16) || !aligned(out, 16)) return SNGGUF_E_ALIGN;
    if (qtype == SNGGUF_TYPE_BF16)
        return sngguf::launch_dequantize_bf16(q, rows, cols, out, out_dtype, static_cast<hipStream_t>(stream));
    return sngguf::launch_dequantize(q, qtype, rows, cols, out, out_dtype, numerics, static_cast<hipStream_t>(stream));
}

namespace {

// Between the decode kernels' 64 rows and a few hundred, a matrix with few 256 x 256 output tiles keeps only a few
// compute units busy in the tile kernels, each for K / 64 steps of about 1.6 us, while the decode kernel streams the
// whole matrix in 10 us + N K / 1.25e12 s per 64 rows (measured: 12288 x 4096 50 us, 4096 x 4096 20 us, 1024 x 4096 19 us) and less for a
// short last chunk.  Row chunks through the decode kernel win where the sum of those stays below the tile kernel's time:
// 4096 x 12288 at 128 rows 102 against 292 us, 4096 x 4096 41 against 102 us; 12288 x 4096 only up to 65 rows or so.
// (Chunks start at multiples of 64 rows, so x, y and the residual keep their 16-byte alignment.)
bool row_chunks_win(int64_t M, int64_t N, int64_t K, int qtype) {
    if (K % 256 != 0 || M > 512) return false;
    const double weights = (double)N * (double)K;
    const double t16 = 8.0 + weights * (double)sngguf_type_size(qtype) / (double)sngguf_block_size(qtype) / 6.2e6;   // us
    const double t64_w = 10.0 + weights / 1.25e6;
    const double t64 = t64_w > 19.0 ? t64_w : 19.0;   // 64 activation rows per 16 weight rows: never below 19 us
    const int64_t full = M / 64, rem = M % 64;
    const double last = rem == 0 ? 0.0 : rem <= 16 ? t16 : t16 + (t64 - t16) * (double)(rem - 16) / 48.0;
    const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
    const double t_tile = (double)((tiles + 255) / 256) * (double)(K / 64) * 1.6;
    return (double)full * t64 + last < 0.9 * t_tile;
}

int linear_impl(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias,
                const void* residual, void* y, int numerics, void* stream) {
    const int rc = check_matmul(x, M, q, qtype, N, K, y, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (residual && !aligned(residual, 16)) return SNGGUF_E_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (qtype == SNGGUF_TYPE_BF16) {
        // plain bf16 rows: the decode-sized kernel up to 16 rows, the tile kernel's dense form beyond (whole K steps,
        // 32-bit activation offsets), else 16 rows at a time
        if (M > 16 && K % 64 == 0 && M * K < ((int64_t)1 << 31))
            return sngguf::launch_gemm(x, M, q, 30, N, K, bias, residual, y, numerics, s);
        const char* xp = static_cast<const char*>(x);
        const char* rp = static_cast<const char*>(residual);
        char* yp = static_cast<char*>(y);
        for (int64_t r0 = 0; r0 < M; r0 += 16) {
            const int64_t rows = M - r0 < 16 ? M - r0 : 16;
            // (with an odd K the rows of x are only 2-byte aligned; the kernel then reads single elements)
            const int rc = sngguf::launch_gemv_bf16(xp + 2 * r0 * K, rows, q, nullptr, N, K, bias, rp ? rp + 2 * r0 * N : nullptr,
                                                    yp + 2 * r0 * N, false, s);
            if (rc != SNGGUF_OK) return rc;
        }
        return SNGGUF_OK;
    }
    // decode-shaped work (weights streamed and decoded once): up to 16 rows always, up to 64 rows when the
    // rows are whole 256-element runs
    if (M <= 16 || (M <= 64 && K % 256 == 0))
        return sngguf::launch_gemv(x, M, q, nullptr, qtype, N, K, bias, residual, y, numerics, false, s);
    if (row_chunks_win(M, N, K, qtype)) {
        // a few hundred rows on a matrix with few output tiles: the decode kernel on 64 rows at a time
        const char* xp = static_cast<const char*>(x);
        const char* rp = static_cast<const char*>(residual);
        char* yp = static_cast<char*>(y);
        for (int64_t r0 = 0; r0 < M; r0 += 64) {
            const int64_t rows = M - r0 < 64 ? M - r0 : 64;
            const int rc = sngguf::launch_gemv(xp + 2 * r0 * K, rows, q, nullptr, qtype, N, K, bias,
                                               rp ? rp + 2 * r0 * N : nullptr, yp + 2 * r0 * N, numerics, false, s);
            if (rc != SNGGUF_OK) return rc;
        }
        return SNGGUF_OK;
    }
    return sngguf::launch_gemm(x, M, q, qtype, N, K, bias, residual, y, numerics, s);
}

}  // namespace

int sngguf_linear(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias, void* y,
                  int numerics, void* stream) {
    return linear_impl(x, M, q, qtype, N, K, bias, nullptr, y, numerics, stream);
}

int sngguf_linear_residual(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias,
                           const void* residual, void* y, int numerics, void* stream) {
    if (!residual && M > 0 && N > 0) return SNGGUF_E_NULLPTR;
    return linear_impl(x, M, q, qtype, N, K, bias, residual, y, numerics, stream);
}

namespace {
// The dense kernel wants whole K steps and 32-bit activation offsets.  One weight pass + the dense kernel beat the
// fused kernels from 65 rows on (measured on the four projection shapes of the 8B model, 65 ... 4096 rows); the
// grouped form decodes two weight sets, which pays from a few hundred rows and enough tiles to occupy the chip.
// How many workgroups share the K range of one 256 x 256 tile.  More slices shorten every workgroup's K loop but each
// adds an fp32 copy of the output that is written and read again; fitted on the k / v, q, gate and down shapes at 128,
// 512 and 4096 rows: time ~ rounds of 256 workgroups x K steps per slice x 1.9 us + slices x 8 M N bytes at 5 TB/s.
int64_t pick_k_slices(int64_t M, int64_t N, int64_t tiles, int64_t ksteps, int64_t room, bool fused_decode) {
    int64_t smax = 256 / tiles;
    if (smax > room) smax = room;
    if (smax > ksteps / 2) smax = ksteps / 2;   // at least two K steps per workgroup
    if (smax > 64) smax = 64;
    if (smax < 2) return 1;
    const double t_step = fused_decode ? 1.9 : 1.65, t_slice = 8.0 * (double)M * (double)N / 5e6;   // us
    int64_t best = 2;
    double best_t = 1e30;
    for (int64_t sl = 2; sl <= smax; sl++) {
        const double t = (double)((ksteps + sl - 1) / sl) * t_step + (double)sl * t_slice;
        if (t < best_t) { best_t = t; best = sl; }
    }
    return best;
}

bool dense_route_fits(int64_t M, int64_t N, int64_t K) {
    (void)N;
    return M >= 65 && K % 64 == 0 && M * K < ((int64_t)1 << 31);
}
bool grouped_dense_route_fits(int64_t M, int64_t N, int64_t K) {
    return M >= 384 && K % 64 == 0 && M * K < ((int64_t)1 << 31) && ((M + 255) / 256) * ((N + 255) / 256) >= 128;
}
}  // namespace

int64_t sngguf_linear_workspace_bytes(int64_t N, int64_t K) { return N > 0 && K > 0 && N < kMaxDim && K < kMaxDim ? 2 * N * K : 0; }

namespace {
int linear_ws_impl(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias, void* y,
                   void* workspace, int64_t workspace_bytes, int numerics, void* stream) {
    const int rc = check_matmul(x, M, q, qtype, N, K, y, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (workspace && !aligned(workspace, 16)) return SNGGUF_E_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // everything that does not fit the dense route runs as sngguf_linear does
    const bool plain = qtype == SNGGUF_TYPE_BF16;   // rows that are bf16 already: no weight pass, the dense kernel reads them
    const bool fits = workspace && dense_route_fits(M, N, K);
    if (!fits) return linear_impl(x, M, q, qtype, N, K, bias, nullptr, y, numerics, stream);
    // Few output tiles (a few hundred rows, or a narrow matrix): a 256 x 256 tile takes as long per K step whether
    // or not the other compute units have work, so K is split over enough workgroups to occupy them, with the fp32
    // partial sums in the workspace.  The formats the large-tile kernel decodes itself need no weight pass then and
    // the whole workspace is free for the sums; the others put them behind the decoded weights if the caller's
    // workspace is that large.
    const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
    const int64_t ksteps = K / 64;
    // (from 4096 rows on the weight pass pays for itself even here: a K step of the dense kernel takes 1.4 us against 2.0 us
    // with the decode in the loop, and sixteen row tiles share one pass - 4096 x 1024 <- 4096: 56 against 61 us, 2048 wide
    // 80 against 92 us; at 512 rows the pass costs more than it saves, 48 against 44 us on 4096 x 4096)
    const bool tile_type = plain || ((qtype == SNGGUF_TYPE_Q8_0 || qtype == SNGGUF_TYPE_Q4_K) && M < 4096);
    const int64_t dense_bytes = tile_type ? 0 : 2 * N * K;
    if (tiles <= 128 && workspace_bytes > dense_bytes) {
        const int64_t room = (workspace_bytes - dense_bytes) / (4 * M * N);
        const int64_t slices = pick_k_slices(M, N, tiles, ksteps, room, tile_type && !plain);
        if (slices >= 2) {
            float* partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + dense_bytes);
            if (tile_type)
                return sngguf::launch_gemm_splitk(x, M, q, plain ? 30 : qtype, N, K, bias, y, partial, (int)slices, numerics, s);
            const int rd = sngguf::launch_dequantize(q, qtype, N, K, workspace, SNGGUF_OUT_BF16, numerics, s);
            if (rd != SNGGUF_OK) return rd;
            return sngguf::launch_gemm_splitk(x, M, workspace, 30, N, K, bias, y, partial, (int)slices, numerics, s);
        }
    }
    if (plain) return linear_impl(x, M, q, qtype, N, K, bias, nullptr, y, numerics, stream);
    // no room for a K split: row chunks through the decode kernel where they beat the few tiles of the dense kernel too
    if (workspace_bytes < 2 * N * K || row_chunks_win(M, N, K, qtype))
        return linear_impl(x, M, q, qtype, N, K, bias, nullptr, y, numerics, stream);
    const int rd = sngguf::launch_dequantize(q, qtype, N, K, workspace, SNGGUF_OUT_BF16, numerics, s);
    if (rd != SNGGUF_OK) return rd;
    return sngguf::launch_gemm_dense(x, M, workspace, N, K, bias, y, s);
}
}  // namespace

int sngguf_linear_ws(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias, void* y,
                     void* workspace, int64_t workspace_bytes, int numerics, void* stream) {
    return linear_ws_impl(x, M, q, qtype, N, K, bias, y, workspace, workspace_bytes, numerics, stream);
}

int64_t sngguf_linear_static_max_outputs(void) { return sngguf::static_scratch_bytes() / 8; }

int sngguf_linear_static(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias, void* y,
                         int numerics, void* stream) {
    const int rc = check_matmul(x, M, q, qtype, N, K, y, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    // two fp32 slices of the output must fit the static area: the smallest K split there is
    if (M * N > sngguf_linear_static_max_outputs()) return SNGGUF_E_TOOLARGE;
    void* scratch = nullptr;
    const int rs = sngguf::static_scratch(&scratch);
    if (rs != SNGGUF_OK) return rs;
    return linear_ws_impl(x, M, q, qtype, N, K, bias, y, scratch, sngguf::static_scratch_bytes(), numerics, stream);
}

int sngguf_gate_up_silu(const void* x, int64_t M, const void* q_gate, const void* q_up, int qtype, int64_t N, int64_t K,
                        void* h, int numerics, void* stream) {
    const int rc = check_matmul(x, M, q_gate, qtype, N, K, h, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (!q_up) return SNGGUF_E_NULLPTR;
    if (!aligned(q_up, 16)) return SNGGUF_E_ALIGN;
    if (M > 16) return SNGGUF_E_BADSHAPE;
    if (qtype == SNGGUF_TYPE_BF16)
        return sngguf::launch_gemv_bf16(x, M, q_gate, q_up, N, K, nullptr, nullptr, h, true, static_cast<hipStream_t>(stream));
    return sngguf::launch_gemv(x, M, q_gate, q_up, qtype, N, K, nullptr, nullptr, h, numerics, true, static_cast<hipStream_t>(stream));
}

int64_t sngguf_gate_up_silu_workspace_bytes(int64_t N, int64_t K) {
    return N > 0 && K > 0 && N < kMaxDim && K < kMaxDim ? 2 * 256 * ((N + 127) / 128) * K : 0;
}

int sngguf_gate_up_silu_ws_fits(int qtype, int64_t M, int64_t N, int64_t K) {
    // the dense kernel's gated epilogue: whole pairs of K steps, output rows of whole 16-byte pieces, 32-bit activation
    // offsets; packed block formats only (plain BF16 rows are not interleaved by a weight pass)
    return known_type(qtype) && qtype != SNGGUF_TYPE_BF16 && M >= 17 && M < kMaxDim && N > 0 && N < kMaxDim && K > 0 &&
           K < kMaxDim && K % 128 == 0 && K % sngguf_block_size(qtype) == 0 && N % 8 == 0 && M * K < ((int64_t)1 << 31);
}

int sngguf_gate_up_silu_ws(const void* x, int64_t M, const void* q_gate, const void* q_up, int qtype, int64_t N, int64_t K,
                           void* h, void* workspace, int64_t workspace_bytes, int numerics, void* stream) {
    if (M >= 0 && M <= 16) return sngguf_gate_up_silu(x, M, q_gate, q_up, qtype, N, K, h, numerics, stream);
    const int rc = check_matmul(x, M, q_gate, qtype, N, K, h, numerics);
    if (rc != SNGGUF_OK || N == 0) return rc;
    if (!q_up || !workspace) return SNGGUF_E_NULLPTR;
    if (!aligned(q_up, 16) || !aligned(workspace, 16)) return SNGGUF_E_ALIGN;
    if (!sngguf_gate_up_silu_ws_fits(qtype, M, N, K)) return qtype == SNGGUF_TYPE_BF16 ? SNGGUF_E_BADTYPE : SNGGUF_E_BADSHAPE;
    if (workspace_bytes < sngguf_gate_up_silu_workspace_bytes(N, K)) return SNGGUF_E_BADSHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rd = sngguf::launch_dequantize_interleaved(q_gate, qtype, N, K, workspace, 0, numerics, s);
    if (rd != SNGGUF_OK) return rd;
    rd = sngguf::launch_dequantize_interleaved(q_up, qtype, N, K, workspace, 1, numerics, s);
    if (rd != SNGGUF_OK) return rd;
    return sngguf::launch_gemm_dense_gated(x, M, workspace, N, K, h, s);
}

int64_t sngguf_lm_head_argmax_workspace_bytes(int64_t M, int64_t N) {
    return M > 0 && N > 0 && M <= 16 && N < kMaxDim ? 8 * M * ((N + 15) / 16) : 0;
}

int sngguf_lm_head_argmax(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K, const void* bias,
                          void* workspace, int64_t* out_index, int numerics, void* stream) {
    const int rc = check_matmul(x, M, q, qtype, N, K, x, numerics);      // (no y here: x stands in for its checks)
    if (rc != SNGGUF_OK || M == 0) return rc;
    if (N == 0 || M > 16 || K % 256 != 0) return SNGGUF_E_BADSHAPE;     // the matrix-core decode kernels only
    if (!out_index) return SNGGUF_E_NULLPTR;
    if (!aligned(out_index, 8)) return SNGGUF_E_ALIGN;
    if (qtype == SNGGUF_TYPE_BF16) return SNGGUF_E_BADTYPE;
    if (!workspace) return SNGGUF_E_NULLPTR;
    if (!aligned(workspace, 16)) return SNGGUF_E_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint64_t* keys = static_cast<uint64_t*>(workspace);
    const int rl = qtype == SNGGUF_TYPE_Q8_0
        ? sngguf::launch_gemv_q8_mfma(x, M, q, nullptr, N, K, bias, nullptr, nullptr, numerics, false, s, nullptr, 0.f, keys)
        : sngguf::launch_gemv_kq_mfma(x, M, q, nullptr, qtype, N, K, bias, nullptr, nullptr, numerics, false, s, nullptr, 0.f, keys);
    if (rl != SNGGUF_OK) return rl;
    return sngguf::launch_argmax_reduce(keys, M, sngguf::gemv_argmax_slots(qtype, M, N), out_index, s);
}

int sngguf_rmsnorm(const void* x, int64_t M, int64_t K, const void* gamma, float eps, void* y, void* stream) {
    if (M < 0 || K <= 0 || M >= kMaxDim || K >= kMaxDim || K % 8 != 0 || !(eps >= 0.f)) return SNGGUF_E_BADSHAPE;
    if (M == 0) return SNGGUF_OK;
    if (!x || !gamma || !y) return SNGGUF_E_NULLPTR;
    if (!aligned(x, 16) || !aligned(gamma, 16) || !aligned(y, 16)) return SNGGUF_E_ALIGN;
    return sngguf::launch_rmsnorm(x, M, K, gamma, eps, y, static_cast<hipStream_t>(stream));
}

int sngguf_rmsnorm_fits(int qtype, int64_t M, int64_t K) {
    // the fused norm works on activations staged in LDS: rows of whole 256-element runs, M (2 K + 64) <= 36 KB
    // (four rows at K = 4096, eight at 2048; with the decode kernels' slabs, and the rows staged twice by a gated pair,
    // that stays within a compute unit's 160 KB for every type)
    return known_type(qtype) && qtype != SNGGUF_TYPE_BF16 && M >= 1 && K > 0 && K < kMaxDim && K % 256 == 0 && M * (2 * K + 64) <= 36864;
}

namespace {
int check_rmsnorm(const void* x, int64_t M, const void* gamma, float eps, const void* q, int qtype, int64_t N, int64_t K,
                  const void* y, int numerics) {
    const int rc = check_matmul(x, M, q, qtype, N, K, y, numerics);
    if (rc != SNGGUF_OK) return rc;
    if (!(eps >= 0.f)) return SNGGUF_E_BADSHAPE;
    if (M == 0 || N == 0) return SNGGUF_OK;
    if (!sngguf_rmsnorm_fits(qtype, M, K)) return SNGGUF_E_BADSHAPE;
    if (!gamma) return SNGGUF_E_NULLPTR;
    if (!aligned(gamma, 16)) return SNGGUF_E_ALIGN;
    return SNGGUF_OK;
}
}  // namespace

int sngguf_rmsnorm_linear(const void* x, int64_t M, const void* gamma, float eps, const void* q, int qtype, int64_t N,
                          int64_t K, const void* bias, void* y, int numerics, void* stream) {
    const int rc = check_rmsnorm(x, M, gamma, eps, q, qtype, N, K, y, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (qtype != SNGGUF_TYPE_Q8_0)
        return sngguf::launch_gemv_kq_mfma(x, M, q, nullptr, qtype, N, K, bias, nullptr, y, numerics, false,
                                           static_cast<hipStream_t>(stream), gamma, eps);
    return sngguf::launch_gemv_q8_mfma(x, M, q, nullptr, N, K, bias, nullptr, y, numerics, false,
                                       static_cast<hipStream_t>(stream), gamma, eps);
}

int sngguf_rmsnorm_gate_up_silu(const void* x, int64_t M, const void* gamma, float eps, const void* q_gate,
                                const void* q_up, int qtype, int64_t N, int64_t K, void* h, int numerics, void* stream) {
    const int rc = check_rmsnorm(x, M, gamma, eps, q_gate, qtype, N, K, h, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (!q_up) return SNGGUF_E_NULLPTR;
    if (!aligned(q_up, 16)) return SNGGUF_E_ALIGN;
    if (qtype != SNGGUF_TYPE_Q8_0)
        return sngguf::launch_gemv_kq_mfma(x, M, q_gate, q_up, qtype, N, K, nullptr, nullptr, h, numerics, true,
                                           static_cast<hipStream_t>(stream), gamma, eps);
    return sngguf::launch_gemv_q8_mfma(x, M, q_gate, q_up, N, K, nullptr, nullptr, h, numerics, true,
                                       static_cast<hipStream_t>(stream), gamma, eps);
}

int64_t sngguf_q8_0_tiled_bytes(int64_t N, int64_t K) {
    if (N <= 0 || K <= 0 || N >= kMaxDim || K >= kMaxDim || K % 256 != 0) return 0;
    return sngguf::q8_0_tiled_bytes(N, K);
}

int sngguf_q8_0_tile(const void* q, int64_t N, int64_t K, void* tiled, void* stream) {
    if (N < 0 || K <= 0 || N >= kMaxDim || K >= kMaxDim || K % 256 != 0) return SNGGUF_E_BADSHAPE;
    if (N == 0) return SNGGUF_OK;
    if (!q || !tiled) return SNGGUF_E_NULLPTR;
    if (!aligned(q, 16) || !aligned(tiled, 16)) return SNGGUF_E_ALIGN;
    return sngguf::launch_q8_0_tile(q, N, K, tiled, static_cast<hipStream_t>(stream));
}

namespace {
int check_tiled(const void* x, int64_t M, const void* t, int64_t N, int64_t K, const void* y, int numerics) {
    if (!known_numerics(numerics)) return SNGGUF_E_BADTYPE;
    if (M < 0 || M > 16 || N < 0 || K <= 0 || N >= kMaxDim || K >= ((int64_t)1 << 27) || K % 256 != 0) return SNGGUF_E_BADSHAPE;  // 32-bit offsets inside a row group
    if (M == 0 || N == 0) return SNGGUF_OK;
    if (!x || !t || !y) return SNGGUF_E_NULLPTR;
    if (!aligned(x, 16) || !aligned(y, 16) || !aligned(t, 16)) return SNGGUF_E_ALIGN;
    return SNGGUF_OK;
}
}  // namespace

int sngguf_linear_tiled(const void* x, int64_t M, const void* tiled, int64_t N, int64_t K, const void* bias,
                        const void* residual, void* y, int numerics, void* stream) {
    const int rc = check_tiled(x, M, tiled, N, K, y, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (residual && !aligned(residual, 16)) return SNGGUF_E_ALIGN;
    return sngguf::launch_gemv_q8_tiled(x, M, tiled, nullptr, N, K, bias, residual, y, numerics, false,
                                        static_cast<hipStream_t>(stream));
}

int sngguf_gate_up_silu_tiled(const void* x, int64_t M, const void* tiled_gate, const void* tiled_up, int64_t N, int64_t K,
                              void* h, int numerics, void* stream) {
    const int rc = check_tiled(x, M, tiled_gate, N, K, h, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (!tiled_up) return SNGGUF_E_NULLPTR;
    if (!aligned(tiled_up, 16)) return SNGGUF_E_ALIGN;
    return sngguf::launch_gemv_q8_tiled(x, M, tiled_gate, tiled_up, N, K, nullptr, nullptr, h, numerics, true,
                                        static_cast<hipStream_t>(stream));
}

namespace {
int check_rmsnorm_tiled(const void* x, int64_t M, const void* gamma, float eps, const void* t, int64_t N, int64_t K,
                        const void* y, int numerics) {
    const int rc = check_tiled(x, M, t, N, K, y, numerics);
    if (rc != SNGGUF_OK) return rc;
    if (!(eps >= 0.f)) return SNGGUF_E_BADSHAPE;
    if (M == 0 || N == 0) return SNGGUF_OK;
    if (!sngguf_rmsnorm_fits(SNGGUF_TYPE_Q8_0, M, K)) return SNGGUF_E_BADSHAPE;
    if (!gamma) return SNGGUF_E_NULLPTR;
    if (!aligned(gamma, 16)) return SNGGUF_E_ALIGN;
    return SNGGUF_OK;
}
}  // namespace

int sngguf_rmsnorm_linear_tiled(const void* x, int64_t M, const void* gamma, float eps, const void* tiled, int64_t N,
                                int64_t K, const void* bias, void* y, int numerics, void* stream) {
    const int rc = check_rmsnorm_tiled(x, M, gamma, eps, tiled, N, K, y, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    return sngguf::launch_gemv_q8_tiled(x, M, tiled, nullptr, N, K, bias, nullptr, y, numerics, false,
                                        static_cast<hipStream_t>(stream), gamma, eps);
}

int sngguf_rmsnorm_gate_up_silu_tiled(const void* x, int64_t M, const void* gamma, float eps, const void* tiled_gate,
                                      const void* tiled_up, int64_t N, int64_t K, void* h, int numerics, void* stream) {
    const int rc = check_rmsnorm_tiled(x, M, gamma, eps, tiled_gate, N, K, h, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (!tiled_up) return SNGGUF_E_NULLPTR;
    if (!aligned(tiled_up, 16)) return SNGGUF_E_ALIGN;
    return sngguf::launch_gemv_q8_tiled(x, M, tiled_gate, tiled_up, N, K, nullptr, nullptr, h, numerics, true,
                                        static_cast<hipStream_t>(stream), gamma, eps);
}

int64_t sngguf_mlp_decode_workspace_bytes(int64_t M, int64_t hidden, int64_t inter) {
    if (M < 1 || M > 16 || hidden <= 0 || inter <= 0 || hidden >= kMaxDim || inter >= kMaxDim) return 0;
    return sngguf::mlp_q8_decode_workspace_bytes(M, inter) + ((2 * M * hidden + 255) & ~(int64_t)255);
}

int64_t sngguf_mlp_decode_status_offset(void) { return sngguf::mlp_q8_decode_status_offset(); }

int sngguf_mlp_decode_fits(int qtype_gate_up, int qtype_down, int64_t M, int64_t hidden, int64_t inter) {
    if (qtype_gate_up == SNGGUF_TYPE_Q8_0 && qtype_down == SNGGUF_TYPE_Q8_0) return sngguf::mlp_q8_decode_fits(M, hidden, inter);
    return sngguf::mlp_kq_decode_fits(qtype_gate_up, qtype_down, M, hidden, inter);
}

int sngguf_mlp_decode(const void* x, int64_t M, const void* gamma, float eps, const void* q_gate, const void* q_up, int qtype_gate_up,
                      const void* q_down, int qtype_down, int64_t hidden, int64_t inter, const void* residual, void* y,
                      void* workspace, int64_t workspace_bytes, int numerics, int spin_limit, void* stream) {
    int rc = check_matmul(x, M, q_gate, qtype_gate_up, inter, hidden, y, numerics);
    if (rc != SNGGUF_OK) return rc;
    rc = check_matmul(x, M, q_down, qtype_down, hidden, inter, y, numerics);
    if (rc != SNGGUF_OK || M == 0 || hidden == 0 || inter == 0) return rc;
    if (M > 16) return SNGGUF_E_BADSHAPE;
    if (!q_up || !workspace) return SNGGUF_E_NULLPTR;
    if (!aligned(q_up, 16) || !aligned(workspace, 256) || (residual && !aligned(residual, 16)) || (gamma && !aligned(gamma, 16)))
        return SNGGUF_E_ALIGN;
    if (gamma && !(eps >= 0.f)) return SNGGUF_E_BADSHAPE;
    if (workspace_bytes < sngguf_mlp_decode_workspace_bytes(M, hidden, inter)) return SNGGUF_E_BADSHAPE;
    if (sngguf_mlp_decode_fits(qtype_gate_up, qtype_down, M, hidden, inter)) {
        if (qtype_gate_up == SNGGUF_TYPE_Q8_0)
            return sngguf::launch_mlp_q8_decode(x, M, gamma, eps, q_gate, q_up, q_down, hidden, inter, residual, y, workspace, numerics,
                                                spin_limit, static_cast<hipStream_t>(stream));
        return sngguf::launch_mlp_kq_decode(x, M, gamma, eps, q_gate, q_up, q_down, qtype_down, hidden, inter, residual, y, workspace,
                                            numerics, spin_limit, static_cast<hipStream_t>(stream));
    }
    // every other shape and type: the same arithmetic as separate launches, the gated activations (and, where the norm
    // does not ride inside the pair's launch, the normalized rows) in the workspace
    char* h = static_cast<char*>(workspace) + sngguf::mlp_q8_decode_ctl_bytes();
    char* xn = static_cast<char*>(workspace) + sngguf::mlp_q8_decode_workspace_bytes(M, inter);
    if (gamma && sngguf_rmsnorm_fits(qtype_gate_up, M, hidden)) {
        rc = sngguf_rmsnorm_gate_up_silu(x, M, gamma, eps, q_gate, q_up, qtype_gate_up, inter, hidden, h, numerics, stream);
    } else {
        if (gamma) {
            rc = sngguf_rmsnorm(x, M, hidden, gamma, eps, xn, stream);
            if (rc != SNGGUF_OK) return rc;
        }
        rc = sngguf_gate_up_silu(gamma ? xn : x, M, q_gate, q_up, qtype_gate_up, inter, hidden, h, numerics, stream);
    }
    if (rc != SNGGUF_OK) return rc;
    return residual ? sngguf_linear_residual(h, M, q_down, qtype_down, hidden, inter, nullptr, residual, y, numerics, stream)
                    : sngguf_linear(h, M, q_down, qtype_down, hidden, inter, nullptr, y, numerics, stream);
}

int64_t sngguf_probe_stream_read_out_bytes(void) { return sngguf::stream_probe_out_bytes(); }

int sngguf_probe_stream_read(const void* p, int64_t bytes, void* out, int workgroups, int nontemporal, void* stream) {
    if (bytes < 0 || workgroups < 0) return SNGGUF_E_BADSHAPE;
    if (bytes == 0) return SNGGUF_OK;
    if (!p || !out) return SNGGUF_E_NULLPTR;
    if (!aligned(p, 16) || !aligned(out, 16)) return SNGGUF_E_ALIGN;
    return sngguf::launch_stream_read(p, bytes, out, workgroups, nontemporal != 0, static_cast<hipStream_t>(stream));
}

int64_t sngguf_grouped_workspace_bytes(int64_t M) { return sngguf::grouped_workspace_bytes(M); }

int sngguf_grouped_linear(const void* x, int64_t M, const uint8_t* indicator, int64_t n_text, const void* q_und,
                          int qtype_und, const void* q_gen, int qtype_gen, int64_t N, int64_t K, const void* bias_und,
                          const void* bias_gen, void* y, void* workspace, int numerics, void* stream) {
    int rc = check_matmul(x, M, q_und, qtype_und, N, K, y, numerics);
    if (rc != SNGGUF_OK) return rc;
    rc = check_matmul(x, M, q_gen, qtype_gen, N, K, y, numerics);
    if (rc != SNGGUF_OK || M == 0 || N == 0) return rc;
    if (indicator) {
        if (!workspace) return SNGGUF_E_NULLPTR;
        if (!aligned(workspace, 16)) return SNGGUF_E_ALIGN;
    } else if (n_text < 0 || n_text > M) {
        return SNGGUF_E_BADSHAPE;
    }
    // plain bf16 rows run on the tile kernel's dense form only: whole K steps, 32-bit activation offsets
    if ((qtype_und == SNGGUF_TYPE_BF16 || qtype_gen == SNGGUF_TYPE_BF16) && (K % 64 != 0 || M * K >= ((int64_t)1 << 31)))
        return SNGGUF_E_BADSHAPE;
    return sngguf::launch_grouped_gemm(x, M, indicator, n_text, q_und, qtype_und, q_gen, qtype_gen, N, K, bias_und,
                                       bias_gen, y, workspace, numerics, static_cast<hipStream_t>(stream));
}

int sngguf_grouped_linear_ws(const void* x, int64_t M, const uint8_t* indicator, int64_t n_text, const void* q_und,
                             int qtype_und, const void* q_gen, int qtype_gen, int64_t N, int64_t K, const void* bias_und,
                             const void* bias_gen, void* y, void* workspace, void* dense_workspace,
                             int64_t dense_workspace_bytes, int numerics, void* stream) {
    // The contiguous [text rows | image rows] layout needs no row map, so the two groups are two plain problems on
    // consecutive row ranges: each takes the route sngguf_linear_ws would pick for its own row count (a few hundred
    // text rows: K split without a weight pass; thousands of image rows: weight pass + dense kernel), one after the
    // other on the stream with the same workspace.  Measured on a 512 + 4096-row layer of seven Q8_0 projections:
    // 1.9 ms against 2.3 ms for one dense launch over both groups, which decodes the understanding weights in full
    // for two row tiles.
    if (!indicator && dense_workspace && n_text >= 0 && n_text <= M && M > 0 && N > 0) {
        int rc = check_matmul(x, M, q_und, qtype_und, N, K, y, numerics);
        if (rc != SNGGUF_OK) return rc;
        rc = check_matmul(x, M, q_gen, qtype_gen, N, K, y, numerics);
        if (rc != SNGGUF_OK) return rc;
        if (!aligned(dense_workspace, 16)) return SNGGUF_E_ALIGN;
        // (a group boundary at an odd row of an odd-width matrix would leave the second group's rows 2-byte aligned)
        const bool split_ok = (2 * n_text * K) % 16 == 0 && (2 * n_text * N) % 16 == 0;
        if (split_ok) {
            const char* xp = static_cast<const char*>(x);
            char* yp = static_cast<char*>(y);
            if (n_text > 0) {
                rc = linear_ws_impl(xp, n_text, q_und, qtype_und, N, K, bias_und, yp, dense_workspace, dense_workspace_bytes, numerics, stream);
                if (rc != SNGGUF_OK) return rc;
            }
            if (n_text < M)
                rc = linear_ws_impl(xp + 2 * n_text * K, M - n_text, q_gen, qtype_gen, N, K, bias_gen, yp + 2 * n_text * N, dense_workspace,
                                    dense_workspace_bytes, numerics, stream);
            return rc;
        }
    }
    const bool two_pass = dense_workspace && dense_workspace_bytes >= 4 * N * K && K > 0 && N > 0 && grouped_dense_route_fits(M, N, K);
    // Few output tiles (narrow matrices such as k / v, or a few hundred rows) of one type the large-tile kernel decodes
    // itself: K split over workgroups, the fp32 partial sums in the dense workspace (as sngguf_linear_ws does)
    const bool tile_types = qtype_und == qtype_gen && (qtype_und == SNGGUF_TYPE_Q8_0 || qtype_und == SNGGUF_TYPE_Q4_K);
    if (!two_pass && dense_workspace && tile_types && M >= 65 && N > 0 && K > 0 && K % 64 == 0 && M < kMaxDim && N < kMaxDim
        && K < kMaxDim && M * K < ((int64_t)1 << 31)) {
        const int64_t tiles = ((M + 255) / 256 + 1) * ((N + 255) / 256);   // a split into two groups adds one partial row tile
        const int64_t room = dense_workspace_bytes / (4 * M * N);
        const int64_t slices = tiles <= 128 ? pick_k_slices(M, N, tiles, K / 64, room, true) : 0;
        if (slices >= 2) {
            int rc = check_matmul(x, M, q_und, qtype_und, N, K, y, numerics);
            if (rc != SNGGUF_OK) return rc;
            rc = check_matmul(x, M, q_gen, qtype_gen, N, K, y, numerics);
            if (rc != SNGGUF_OK) return rc;
            if (!aligned(dense_workspace, 16)) return SNGGUF_E_ALIGN;
            if (indicator) {
                if (!workspace) return SNGGUF_E_NULLPTR;
                if (!aligned(workspace, 16)) return SNGGUF_E_ALIGN;
            } else if (n_text < 0 || n_text > M) {
                return SNGGUF_E_BADSHAPE;
            }
            return sngguf::launch_grouped_gemm(x, M, indicator, n_text, q_und, qtype_und, q_gen, qtype_gen, N, K, bias_und,
                                               bias_gen, y, workspace, numerics, static_cast<hipStream_t>(stream),
                                               static_cast<float*>(dense_workspace), (int)slices);
        }
    }
    if (!two_pass)
        return sngguf_grouped_linear(x, M, indicator, n_text, q_und, qtype_und, q_gen, qtype_gen, N, K, bias_und, bias_gen, y,
                                     workspace, numerics, stream);
    int rc = check_matmul(x, M, q_und, qtype_und, N, K, y, numerics);
    if (rc != SNGGUF_OK) return rc;
    rc = check_matmul(x, M, q_gen, qtype_gen, N, K, y, numerics);
    if (rc != SNGGUF_OK) return rc;
    if (!aligned(dense_workspace, 16)) return SNGGUF_E_ALIGN;
    if (indicator) {
        if (!workspace) return SNGGUF_E_NULLPTR;
        if (!aligned(workspace, 16)) return SNGGUF_E_ALIGN;
    } else if (n_text < 0 || n_text > M) {
        return SNGGUF_E_BADSHAPE;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint8_t* w_und = static_cast<uint8_t*>(dense_workspace);
    uint8_t* w_gen = w_und + 2 * N * K;
    rc = qtype_und == SNGGUF_TYPE_BF16 ? sngguf::launch_dequantize_bf16(q_und, N, K, w_und, SNGGUF_OUT_BF16, s)
                                       : sngguf::launch_dequantize(q_und, qtype_und, N, K, w_und, SNGGUF_OUT_BF16, numerics, s);
    if (rc != SNGGUF_OK) return rc;
    rc = qtype_gen == SNGGUF_TYPE_BF16 ? sngguf::launch_dequantize_bf16(q_gen, N, K, w_gen, SNGGUF_OUT_BF16, s)
                                       : sngguf::launch_dequantize(q_gen, qtype_gen, N, K, w_gen, SNGGUF_OUT_BF16, numerics, s);
    if (rc != SNGGUF_OK) return rc;
    return sngguf::launch_grouped_gemm(x, M, indicator, n_text, w_und, 30, w_gen, 30, N, K, bias_und, bias_gen, y, workspace,
                                       numerics, s);
}

}  // extern "C"
