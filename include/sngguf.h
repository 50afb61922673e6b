/*
 * sngguf.h - C ABI of the MI355X (gfx950) GGUF quantized-linear library.
 *
 * Every entry point takes plain device pointers and sizes, enqueues its work on
 * the HIP stream it is given (a hipStream_t passed as void*, NULL = the null
 * stream), never synchronises, never allocates and never throws.  The return
 * value is SNGGUF_OK or a negative SNGGUF_E_* code; sngguf_strerror() turns it
 * into text.  Buffers are borrowed for the duration of the enqueue only: the
 * caller keeps them alive by stream ordering.
 *
 * The reference (OpenSenseNova/SenseNova-U1) has no native code on this path;
 * its arithmetic lives in the third-party packages it imports at
 * src/sensenova_u1/utils/gguf_loader.py:24,29-33,64-66 (diffusers 0.37.1
 * quantizers/gguf/utils.py, gguf 0.19.0).  Each declaration below names the
 * Python-level interface it stands in for.
 */
#ifndef SNGGUF_H
#define SNGGUF_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml tensor type numbers (gguf.GGMLQuantizationType, the `quant_type` that
 * src/sensenova_u1/utils/gguf_loader.py:37-43 stores on each GGUFParameter). */
enum {
    SNGGUF_TYPE_Q4_0 = 2,  /* 32 elements / 18 bytes:  f16 d; u8 qs[16]                          */
    SNGGUF_TYPE_Q4_1 = 3,  /* 32 elements / 20 bytes:  f16 d, m; u8 qs[16]                       */
    SNGGUF_TYPE_Q5_0 = 6,  /* 32 elements / 22 bytes:  f16 d; u8 qh[4]; u8 qs[16]                */
    SNGGUF_TYPE_Q5_1 = 7,  /* 32 elements / 24 bytes:  f16 d, m; u8 qh[4]; u8 qs[16]             */
    SNGGUF_TYPE_Q8_0 = 8,  /* 32 elements / 34 bytes:  f16 d; i8 qs[32]                         */
    SNGGUF_TYPE_Q2_K = 10, /* 256 elements / 84 bytes:  u8 scales[16]; u8 qs[64]; f16 d, dmin    */
    SNGGUF_TYPE_Q3_K = 11, /* 256 elements / 110 bytes: u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d */
    SNGGUF_TYPE_Q4_K = 12, /* 256 elements / 144 bytes: f16 d, dmin; u8 scales[12]; u8 qs[128]  */
    SNGGUF_TYPE_Q5_K = 13, /* 256 elements / 176 bytes: f16 d, dmin; u8 scales[12]; u8 qh[32]; u8 qs[128] */
    SNGGUF_TYPE_Q6_K = 14, /* 256 elements / 210 bytes: u8 ql[128]; u8 qh[64]; i8 sc[16]; f16 d */
    SNGGUF_TYPE_BF16 = 30  /* 1 element / 2 bytes: plain bfloat16 rows (upstream wraps BF16 tensors in a GGUFParameter
                              too and decodes them with dequantize_blocks_BF16: exact in either numerics mode).  Taken by
                              sngguf_dequantize, sngguf_linear[_residual | _ws], sngguf_gate_up_silu and, with
                              K % 64 == 0, the grouped launchers; not by the fused-norm and tiled-layout entry points */
};

/* element type of the `out` buffer of sngguf_dequantize */
enum {
    SNGGUF_OUT_F32 = 0,
    SNGGUF_OUT_F16 = 1,
    SNGGUF_OUT_BF16 = 2
};

/*
 * Rounding chain of the block decode.
 *  SNGGUF_NUM_GGML_FP32      exact fp32 decode (ggml dequantize_row_* semantics), rounded
 *                            once when a narrower type is asked for.
 *  SNGGUF_NUM_UPSTREAM_FP16  replays diffusers' dequantize_blocks_* called with dtype=None:
 *                            every tensor op of that decode is an fp16 op (computed in fp32,
 *                            rounded to fp16, round-to-nearest-even, subnormals kept), and the
 *                            fp16 weight is then cast to the compute dtype.  This is what
 *                            GGUFLinear.forward_native feeds to F.linear, so it is the mode a
 *                            drop-in uses.
 */
enum {
    SNGGUF_NUM_GGML_FP32 = 0,
    SNGGUF_NUM_UPSTREAM_FP16 = 1
};

enum {
    SNGGUF_OK = 0,
    SNGGUF_E_BADTYPE = -1,   /* qtype / out_dtype / numerics not one of the enums above       */
    SNGGUF_E_BADSHAPE = -2,  /* negative size, cols % block != 0, size beyond kernel limits   */
    SNGGUF_E_NULLPTR = -3,   /* a required pointer is NULL                                    */
    SNGGUF_E_ALIGN = -4,     /* a pointer violates the alignment stated for it                */
    SNGGUF_E_LAUNCH = -5,    /* the HIP runtime refused the launch (hipGetLastError != 0)     */
    SNGGUF_E_NODEVICE = -6,  /* no usable gfx950 device / code object                         */
    SNGGUF_E_IO = -7,        /* a file could not be opened or mapped                          */
    SNGGUF_E_FORMAT = -8,    /* not a GGUF file, truncated, corrupt, or a tensor type of unknown size */
    SNGGUF_E_TOOLARGE = -9   /* sngguf_linear_static: M * N beyond sngguf_linear_static_max_outputs()         */
};

/* Library version (major*10000 + minor*100 + patch) and error text. */
int sngguf_version(void);
const char* sngguf_strerror(int code);

/* Bytes per block and elements per block of a ggml type (gguf.GGML_QUANT_SIZES);
 * 0 for a type this library does not decode. */
int64_t sngguf_type_size(int qtype);
int64_t sngguf_block_size(int qtype);

/*
 * Standalone dequantize.  Replaces diffusers.quantizers.gguf.utils.dequantize_gguf_tensor
 * (+ dequantize_blocks_Q8_0 / _Q4_K / _Q5_K / _Q6_K), the function GGUFLinear.forward_native calls
 * on the GGUFParameter built at src/sensenova_u1/utils/gguf_loader.py:43, and the upstream
 * operator seam ops.ggml_dequantize(qweight, qtype, rows, cols).
 *
 *  q      packed blocks, row-major [rows][cols / block * type_size] bytes, base 16-byte aligned
 *  out    [rows][cols] elements of out_dtype, base 16-byte aligned
 * With SNGGUF_OUT_F32 + SNGGUF_NUM_GGML_FP32 the result is the exact ggml value; with
 * SNGGUF_OUT_F16 + SNGGUF_NUM_UPSTREAM_FP16 it is bit-identical to the upstream fp16 tensor.
 */
int sngguf_dequantize(const void* q, int qtype, int64_t rows, int64_t cols,
                      void* out, int out_dtype, int numerics, void* stream);

/*
 * y[M][N] = x[M][K] . dequant(q)[N][K]^T (+ bias[N]).  Replaces GGUFLinear.forward
 * (diffusers quantizers/gguf/utils.py: dequantize -> .to(compute_dtype) -> F.linear), i.e.
 * what every `module(x)` call at src/sensenova_u1/models/neo_unify/modeling_qwen3.py:214-216,
 * 444,450,456,504,602,608,614,709,744 executes once the loader has swapped the module.
 *
 *  x, y, bias   bf16, row-major, x and y 16-byte aligned, bias may be NULL
 *  q            packed blocks [N][K / block * type_size], base 16-byte aligned (rows follow each
 *               other without padding, as in a GGUF file)
 * The weight is rounded to bf16 exactly as `numerics` says, products are accumulated in
 * fp32, bias is added in fp32 and the sum is rounded once to bf16.  M <= 16 takes the fused
 * dequant-GEMV (packed bytes streamed once, nothing dequantized is written to memory);
 * larger M takes the LDS-staged dequant-GEMM on bf16 MFMA.
 * Rows beyond the decode kernels' 64 go to the tile GEMM kernels, except that a few hundred rows on a matrix with few
 * 256 x 256 output tiles (K % 256 == 0) run as 64-row chunks through the decode kernel where that is faster.
 */
int sngguf_linear(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K,
                  const void* bias, void* y, int numerics, void* stream);

/*
 * residual + linear: y[M][N] = bf16(residual[M][N] + bf16(x . W^T + bias)) - the decoder layer's
 * `hidden_states = residual + o_proj(attn)` and `residual + mlp(...)`
 * (src/sensenova_u1/models/neo_unify/modeling_qwen3.py:934,940,973,979) with the add folded into the
 * projection's epilogue, rounding after the projection and after the add as the two separate bf16
 * tensor operations do.  residual: bf16 [M][N], 16-byte aligned, must not overlap y.  Everything
 * else as sngguf_linear.
 */
int sngguf_linear_residual(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K,
                           const void* bias, const void* residual, void* y, int numerics, void* stream);

/*
 * sngguf_linear with a caller-provided workspace.  No counterpart in the reference, whose forward_native
 * materialises the dequantized weight on every call (diffusers GGUFLinear.forward_native, reached from
 * src/sensenova_u1/utils/gguf_loader.py:64-81): this is that route for callers of the bare ABI.  With
 * workspace (device memory, 16-byte aligned) of at least sngguf_linear_workspace_bytes(N, K) = 2 N K bytes
 * and a problem it fits (M >= 65, K % 64 == 0, M K < 2^31) the weights are decoded once into the workspace as bf16 - the same values, same rounding chain,
 * as the fused kernels decode on the fly - and a dense bf16 tile GEMM consumes them; any of the ten types then
 * runs at the rate of that GEMM.  A problem with at most 128 output tiles of 256 x 256 (a few hundred rows, or a
 * narrow matrix) is split along K over floor(256 / tiles) workgroups per tile, with fp32 partial sums in the
 * workspace and a second pass that adds them: Q8_0 and Q4_K then skip the weight pass and use the 2 N K bytes
 * for the sums, the other types need 4 S M N bytes more than 2 N K for it.  Otherwise (workspace NULL or too
 * small included) it behaves exactly as sngguf_linear.  The workspace holds nothing the caller needs afterwards; calls sharing one workspace must
 * be ordered on one stream.  Never allocates.
 */
int64_t sngguf_linear_workspace_bytes(int64_t N, int64_t K);
int sngguf_linear_ws(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K,
                     const void* bias, void* y, void* workspace, int64_t workspace_bytes, int numerics,
                     void* stream);

/*
 * sngguf_linear_ws without a workspace argument and without any allocation.  No counterpart in the reference:
 * it exists for callers that cannot allocate device memory - code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc - and therefore cannot hand sngguf_linear_ws a workspace, yet want its K split
 * for problems with few output tiles.  The workspace is a 64 MiB array inside the library's own device image
 * (one copy per GPU, held until the process ends); the result is bit-identical to sngguf_linear_ws called with a
 * 64 MiB workspace.
 *
 * Limit: M * N <= sngguf_linear_static_max_outputs() (= 8 Mi outputs: two fp32 slices of the output fit), else
 * SNGGUF_E_TOOLARGE; such problems have enough tiles for sngguf_linear.
 * The first call on a device looks up the array's address on that device (hipGetSymbolAddress) and caches it;
 * make that call before a capture begins.  No call allocates or frees.  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (different streams) race; calls on one stream are ordered.
 */
int64_t sngguf_linear_static_max_outputs(void);
int sngguf_linear_static(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K,
                         const void* bias, void* y, int numerics, void* stream);

/*
 * The SiLU-gated MLP of a decoder layer for up to 16 rows:
 *     y = [residual +] down(silu(gate(n)) * up(n)),   n = RMSNorm(x; gamma, eps) if gamma else x
 * i.e. Qwen3MLP.forward (src/sensenova_u1/models/neo_unify/modeling_qwen3.py:214-216) with, optionally, the
 * post_attention_layernorm in front of it and the residual add behind it (Qwen3DecoderLayer.forward, :936-941), every
 * rounding of the separate bf16 tensor operations kept.  x, y, residual [M][hidden], gamma [hidden] bf16;
 * q_gate, q_up [inter][hidden], q_down [hidden][inter] packed.
 *
 * Where sngguf_mlp_decode_fits() says so (Q8_0 for all three, or Q4_K gate / up with a Q6_K or Q4_K down projection;
 * hidden 4096, inter 12288, M <= 2, one compute unit per 48-row slice of gate / up) the whole MLP is ONE launch: every workgroup computes its slice of the gated activations,
 * hands them to the others through the workspace (8-byte words that carry the launch's generation tag beside the data)
 * and goes on with 16 rows of the down projection as the slices it needs arrive; the down weights are requested while
 * the slower workgroups still finish.  All workgroups of that launch must be resident
 * together, which a device that runs nothing else at that moment guarantees.  The wait for the other workgroups is
 * bounded (`spin_limit` polls of about a microsecond; 0 = 2^20, negative = give up at once): on giving up a workgroup
 * sets the 32-bit word at byte sngguf_mlp_decode_status_offset() of the workspace to 1, finishes with whatever the
 * activations hold and the launch ends normally - the caller reads that word when it synchronises, and the results
 * of a call that set it are void.  Everything else runs as the separate launches of sngguf_[rmsnorm_]gate_up_silu
 * and sngguf_linear[_residual] with the activations in the workspace: same values.  (The one launch against the
 * separate ones: equal up to the order in which fp32 partial sums are added - the down projection's K split and, for
 * the K-quant mixes with gamma, the sum of squares.)
 *
 * workspace: sngguf_mlp_decode_workspace_bytes(M, hidden, inter) bytes, 256-byte aligned, all zero before the first
 * call and the launches' own from then on (generation counter and tagged words; never cleared again, also not
 * between replays of a captured graph).  One workspace serves one stream: calls that overlap in time on one
 * workspace, or two one-launch calls that overlap on one device, can starve each other of compute units and time out.
 */
int64_t sngguf_mlp_decode_workspace_bytes(int64_t M, int64_t hidden, int64_t inter);
int64_t sngguf_mlp_decode_status_offset(void);
int sngguf_mlp_decode_fits(int qtype_gate_up, int qtype_down, int64_t M, int64_t hidden, int64_t inter);
int sngguf_mlp_decode(const void* x, int64_t M, const void* gamma, float eps, const void* q_gate, const void* q_up,
                      int qtype_gate_up, const void* q_down, int qtype_down, int64_t hidden, int64_t inter,
                      const void* residual, void* y, void* workspace, int64_t workspace_bytes, int numerics,
                      int spin_limit, void* stream);

/*
 * Measurement aid, no counterpart in the reference: one launch that reads `bytes` (rounded down to 16) of device
 * memory once - contiguous shares per workgroup, 16 bytes per lane and request, eight requests in flight per lane,
 * with (nontemporal != 0) or without the read-once cache hint - and folds them into one word per workgroup in `out`
 * (sngguf_probe_stream_read_out_bytes() bytes, 16-byte aligned).  `workgroups` 0 = 1024 (at most 4096).  Timed over
 * a buffer larger than the last-level cache it gives the read rate this device sustains for a launch of that size,
 * the ceiling the decode kernels' achieved GB/s can be read against beside the published peak.
 */
int64_t sngguf_probe_stream_read_out_bytes(void);
int sngguf_probe_stream_read(const void* p, int64_t bytes, void* out, int workgroups, int nontemporal, void* stream);

/*
 * lm_head followed by torch.argmax: out_index[m] = argmax_n bf16(x[m] . W[n]^T + bias[n]), the greedy next token of
 * the think loop (`torch.argmax(outputs.logits[:, -1, :], dim=-1)`, src/sensenova_u1/models/neo_unify/
 * modeling_neo_chat.py:557,586, on the logits of `self.lm_head(...)`, modeling_qwen3.py:1264).  The decode kernel's
 * epilogue keeps one (value, column) candidate per workgroup and activation row instead of storing N logits; a second
 * small launch picks the winner.  Values compare as the bf16 logits the reference would have stored; among equal
 * values the lowest column wins, a NaN counts as the largest value (torch.argmax's rules).
 *
 *  M <= 16, K % 256 == 0, any of the ten block types (not BF16); anything else is SNGGUF_E_BADSHAPE / _BADTYPE and
 *  the caller runs sngguf_linear + its own arg-max.
 *  workspace   device scratch of sngguf_lm_head_argmax_workspace_bytes(M, N) = 8 M ceil(N / 16) bytes, 16-byte aligned
 *  out_index   int64[M] on the device
 */
int64_t sngguf_lm_head_argmax_workspace_bytes(int64_t M, int64_t N);
int sngguf_lm_head_argmax(const void* x, int64_t M, const void* q, int qtype, int64_t N, int64_t K,
                          const void* bias, void* workspace, int64_t* out_index, int numerics, void* stream);

/*
 * SiLU-gated pair for the decode MLP: h[M][N] = silu(x.Wg^T) * (x.Wu^T), with both
 * projections rounded to bf16 first, silu evaluated in fp32 on the rounded gate and rounded
 * to bf16, and the product rounded to bf16 - the rounding chain of
 * `self.act_fn(self.gate_proj(x)) * self.up_proj(x)` at
 * src/sensenova_u1/models/neo_unify/modeling_qwen3.py:215.  Both weights share qtype, N, K.
 * M <= 16 only (decode); larger M returns SNGGUF_E_BADSHAPE.
 */
int sngguf_gate_up_silu(const void* x, int64_t M, const void* q_gate, const void* q_up, int qtype,
                        int64_t N, int64_t K, void* h, int numerics, void* stream);

/*
 * The same pair beyond decode sizes (the generation tower's thousands of image rows through Qwen3MLP.forward,
 * modeling_qwen3.py:214-216): one weight pass per matrix into the workspace - bf16 rows, the two matrices interleaved
 * in blocks of 128 rows - and ONE launch of the dense tile kernel whose epilogue rounds the gate and the up sums to
 * bf16, applies silu and multiplies, with the roundings above.  The two [M][N] projection outputs are never written
 * and no elementwise pass reads them back.  Same values as sngguf_linear_ws on each matrix followed by
 * silu(gate) * up on bf16 tensors (up to the last place of exp()).
 *  workspace   device scratch of at least sngguf_gate_up_silu_workspace_bytes(N, K) = 512 ceil(N / 128) K bytes,
 *              16-byte aligned; nothing in it outlives the call
 *  M <= 16 runs sngguf_gate_up_silu (the workspace is not touched).  Otherwise the shape must satisfy
 *  sngguf_gate_up_silu_ws_fits(qtype, M, N, K) (M >= 17, K % 128 == 0, N % 8 == 0, M K < 2^31, a packed block
 *  format), else SNGGUF_E_BADSHAPE / SNGGUF_E_BADTYPE and the caller runs the two projections separately.  It
 *  pays from about 512 rows on when the launch's ceil(M / 256) x ceil(N / 128) tiles come close to whole rounds of
 *  the 256 compute units (there is no K split; 12288 x 4096 at
 *  4096 rows: 628 us against 695 us for two sngguf_linear_ws launches and the product, at 2048 rows 354 against 451).
 */
int64_t sngguf_gate_up_silu_workspace_bytes(int64_t N, int64_t K);
int sngguf_gate_up_silu_ws_fits(int qtype, int64_t M, int64_t N, int64_t K);
int sngguf_gate_up_silu_ws(const void* x, int64_t M, const void* q_gate, const void* q_up, int qtype,
                           int64_t N, int64_t K, void* h, void* workspace, int64_t workspace_bytes,
                           int numerics, void* stream);

/*
 * RMSNorm fused in front of a decode projection.  In the decoder layer the q / k / v projections read
 * input_layernorm(hidden) and gate / up read post_attention_layernorm(hidden)
 * (src/sensenova_u1/models/neo_unify/modeling_qwen3.py:919, :938; Qwen3RMSNorm.forward at :192-197):
 *     v = bf16( x * rsqrt(mean(x^2) + eps) )      fp32 arithmetic, one rounding
 *     n = bf16( gamma * v )                       gamma: the norm's weight, K bf16 values, 16-byte aligned
 * and these two entry points contract n instead of x, applying the norm to the activations a workgroup has
 * staged in LDS - no launch and no buffer for the normalized rows.  Offered where that staging exists
 * (sngguf_rmsnorm_fits: any of the ten types, K % 256 == 0, M (2 K + 64) <= 36864, i.e. four rows at K = 4096,
 * eight at 2048); other sizes return SNGGUF_E_BADSHAPE and the caller runs the norm on its own.
 * The sum of squares is added up in a different order than torch's mean, so a normalized value can differ
 * from the reference's by one bf16 unit where the rounding is a near tie; everything after is the same chain
 * as sngguf_linear / sngguf_gate_up_silu.
 */
int sngguf_rmsnorm_fits(int qtype, int64_t M, int64_t K);
/* The same norm as a launch of its own, y[M][K] = RMSNorm(x[M][K]; gamma, eps) (Qwen3RMSNorm.forward,
 * src/sensenova_u1/models/neo_unify/modeling_qwen3.py:192-197), for the row counts the fused entry points do not
 * take: bf16, 16-byte aligned, K % 8 == 0, y may be x. */
int sngguf_rmsnorm(const void* x, int64_t M, int64_t K, const void* gamma, float eps, void* y, void* stream);
int sngguf_rmsnorm_linear(const void* x, int64_t M, const void* gamma, float eps, const void* q, int qtype,
                          int64_t N, int64_t K, const void* bias, void* y, int numerics, void* stream);
int sngguf_rmsnorm_gate_up_silu(const void* x, int64_t M, const void* gamma, float eps, const void* q_gate,
                                const void* q_up, int qtype, int64_t N, int64_t K, void* h, int numerics,
                                void* stream);
/* The same two on the operand-order ("tiled") copy of Q8_0 weights described below (sngguf_q8_0_tile); the size
 * rule is sngguf_rmsnorm_fits(SNGGUF_TYPE_Q8_0, M, K). */
int sngguf_rmsnorm_linear_tiled(const void* x, int64_t M, const void* gamma, float eps, const void* tiled,
                                int64_t N, int64_t K, const void* bias, void* y, int numerics, void* stream);
int sngguf_rmsnorm_gate_up_silu_tiled(const void* x, int64_t M, const void* gamma, float eps,
                                      const void* tiled_gate, const void* tiled_up, int64_t N, int64_t K, void* h,
                                      int numerics, void* stream);

/*
 * Operand-order ("tiled") copy of a Q8_0 matrix for the decode path.  No counterpart in the reference, which keeps
 * the GGUF rows as they are in the file (src/sensenova_u1/utils/gguf_loader.py:42) - and so do all entry points
 * above.  For a model that stays resident on the device a second arrangement of the same blocks, made once at
 * load time, lets the decode GEMV load the weights in the order its matrix instruction consumes them (no staging,
 * no realignment of 34-byte blocks): measured 8 - 10 % faster on the M = 1 MLP step.
 *
 *   sngguf_q8_0_tiled_bytes(N, K)   size of the copy (N rows padded to a multiple of 16; 34 bytes per block as before);
 *                                   0 unless K % 256 == 0
 *   sngguf_q8_0_tile                GGUF Q8_0 rows [N][K / 32 * 34] -> tiled (device to device, on `stream`)
 *   sngguf_linear_tiled             y[M][N] = x[M][K] . W^T (+ bias) (+ residual, as sngguf_linear_residual), 1 <= M <= 16
 *   sngguf_gate_up_silu_tiled       as sngguf_gate_up_silu on two tiled matrices
 * Results are those of sngguf_linear / sngguf_gate_up_silu on the GGUF rows (same decode and rounding chain; the
 * summation order over K differs, as it does between the other kernels).  M > 16 returns SNGGUF_E_BADSHAPE: larger
 * inputs go through the GGUF-native entry points.
 */
int64_t sngguf_q8_0_tiled_bytes(int64_t N, int64_t K);
int sngguf_q8_0_tile(const void* q, int64_t N, int64_t K, void* tiled, void* stream);
int sngguf_linear_tiled(const void* x, int64_t M, const void* tiled, int64_t N, int64_t K, const void* bias,
                        const void* residual, void* y, int numerics, void* stream);
int sngguf_gate_up_silu_tiled(const void* x, int64_t M, const void* tiled_gate, const void* tiled_up,
                              int64_t N, int64_t K, void* h, int numerics, void* stream);

/*
 * Modality-grouped linear: rows of x whose indicator is 0 use the understanding weights
 * q_und, rows whose indicator is non-zero use the generation weights q_gen, in one pass:
 *     y[~ind] = x[~ind] . W_und^T ;  y[ind] = x[ind] . W_gen^T
 * which is the result the mixed branch spells out at
 * src/sensenova_u1/models/neo_unify/modeling_qwen3.py:779-783 (and 802-806, 825-829,
 * 879-883, 1036-1041).
 *
 *  indicator    M bytes (0 / non-zero), or NULL: then rows [0, n_text) are text rows and
 *               rows [n_text, M) are image rows (the contiguous [text | image] layout)
 *  workspace    device scratch of at least sngguf_grouped_workspace_bytes(M) bytes, 16-byte
 *               aligned; may be NULL when indicator is NULL
 *  bias_und / bias_gen   bf16 [N] or NULL
 */
int64_t sngguf_grouped_workspace_bytes(int64_t M);
int sngguf_grouped_linear(const void* x, int64_t M, const uint8_t* indicator, int64_t n_text,
                          const void* q_und, int qtype_und, const void* q_gen, int qtype_gen,
                          int64_t N, int64_t K, const void* bias_und, const void* bias_gen,
                          void* y, void* workspace, int numerics, void* stream);

/*
 * sngguf_grouped_linear with the weight-pass route of sngguf_linear_ws (no counterpart in the reference either):
 * with dense_workspace (device memory, 16-byte aligned) of at least 2 * sngguf_linear_workspace_bytes(N, K) =
 * 4 N K bytes and a problem that fits that route (same conditions as sngguf_linear_ws) both weight sets are
 * decoded into it once as bf16 and ONE dense tile-GEMM launch serves both row groups - whatever the two quant
 * types are.  Otherwise it is sngguf_grouped_linear.  workspace is the row-map scratch of
 * sngguf_grouped_linear (needed with an indicator).  Never allocates.
 * Two weight sets of one type among Q8_0 / Q4_K with at most 128 output tiles (narrow matrices such as k / v, or a
 * few hundred rows) are split along K as sngguf_linear_ws does, the fp32 partial sums in dense_workspace (room for
 * at least two slices of M N floats enables it; the weights are then decoded on the fly).
 */
int sngguf_grouped_linear_ws(const void* x, int64_t M, const uint8_t* indicator, int64_t n_text,
                             const void* q_und, int qtype_und, const void* q_gen, int qtype_gen,
                             int64_t N, int64_t K, const void* bias_und, const void* bias_gen, void* y,
                             void* workspace, void* dense_workspace, int64_t dense_workspace_bytes,
                             int numerics, void* stream);

/*
 * ---- GGUF container reader (host only, no GPU call) -----------------------------------
 * What the reference gets from gguf.GGUFReader at
 * src/sensenova_u1/utils/gguf_loader.py:29-44: open the file, walk `reader.tensors`, read each
 * tensor's name, ggml type and shape, and copy its bytes out of the file mapping (`:42`).
 * The file is mapped read-only; header, metadata and tensor infos (GGUF v2 / v3) are parsed
 * with a bounds check on every read, so a truncated or corrupt file gives SNGGUF_E_FORMAT,
 * never a fault.  `data` / `value` pointers and strings stay valid until sngguf_file_close.
 */
typedef struct sngguf_file sngguf_file;

typedef struct sngguf_tensor_info {
    const char* name;     /* the state-dict key, NUL-terminated                              */
    int32_t ggml_type;    /* GGMLQuantizationType number                                     */
    int32_t n_dims;       /* 0..4                                                            */
    int64_t dims[4];      /* ggml order: dims[0] is the row length (in_features); unused = 1 */
    int64_t n_elements;
    int64_t n_bytes;      /* n_elements / block * type_size                                  */
    int64_t file_offset;  /* of the payload, from the start of the file                      */
    const void* data;     /* the payload inside the read-only mapping                        */
} sngguf_tensor_info;

typedef struct sngguf_metadata_info {
    const char* key;
    int32_t value_type;   /* GGUF value type: 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool,
                             8 string, 9 array, 10 u64, 11 i64, 12 f64                        */
    int32_t item_type;    /* arrays: value type of the items; otherwise -1                   */
    int64_t count;        /* arrays: number of items; strings: byte length; scalars: 1       */
    const void* value;    /* the encoded value as it stands in the file (little endian;
                             strings and arrays start with their length words)               */
    int64_t value_bytes;  /* encoded length of the value                                     */
} sngguf_metadata_info;

/* Opens, maps and parses `path`.  On failure *out is NULL, the return value is negative and
 * `err` (if not NULL, `err_len` bytes) receives a NUL-terminated message. */
int sngguf_file_open(const char* path, sngguf_file** out, char* err, int64_t err_len);
void sngguf_file_close(sngguf_file* f);
int sngguf_file_version(const sngguf_file* f);
int64_t sngguf_file_alignment(const sngguf_file* f);   /* general.alignment, default 32 */
int64_t sngguf_file_tensor_count(const sngguf_file* f);
int sngguf_file_tensor(const sngguf_file* f, int64_t index, sngguf_tensor_info* out);
int64_t sngguf_file_metadata_count(const sngguf_file* f);
int sngguf_file_metadata(const sngguf_file* f, int64_t index, sngguf_metadata_info* out);
/* Copies the payloads of `count` tensors (file order numbers in `indices`) to dst[i], each of at
 * least n_bytes, with up to `threads` threads working on 8 MiB pieces: the copy at
 * gguf_loader.py:42, into buffers the caller chose (pinned host memory, for instance). */
int sngguf_file_read_tensors(const sngguf_file* f, const int64_t* indices, void* const* dst,
                             int64_t count, int threads);

#ifdef __cplusplus
}
#endif
#endif /* SNGGUF_H */
