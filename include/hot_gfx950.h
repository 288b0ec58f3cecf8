/*
 * libhot_gfx950 -- C ABI of the MI355X-native HOT linear-layer backward path.
 *
 * Plain pointers and sizes only; every pointer named "device" must point to
 * memory of the current HIP device.  Every function returns 0 on success or a
 * negative hot_status; hot_last_error() gives the message of the last failure
 * on the calling thread.  No function allocates or frees device memory and
 * none synchronises the stream, except hot_linear_backward() when it is asked
 * for stage timings.
 *
 * What each entry point replaces in the reference (sungonuni/HOT):
 *   hot_hq_rowwise       fwht_kernel + find_scale_kernel + quant_int4_kernel /
 *                        quant_int4_per_token_kernel / quant_int8_kernel
 *                        (cuda_measure/HLQ_backward_kernel.cu:39-178,282-307);
 *                        numerics of lowering_matmul_front + *_quantizer_BWD
 *                        (utils/hadamard_matmul.py:121-141,
 *                         utils/quant_matmul.py:19-31,86-116)
 *   hot_hla_tokenwise    lowering_matmul_back(P, .) + quantiser + the
 *                        transposes feeding the int8 GEMM
 *                        (utils/hadamard_matmul.py:143-161,209-226;
 *                         utils/quant_matmul.py:190,197-198,301,307-320;
 *                         HLQ_backward_kernel.cu:539-543,593-596,607-611)
 *   hot_wq_colwise       lowering_matmul_back(H_n, W) + quantiser + W^T pack
 *                        (utils/quant_matmul.py:270,276-285;
 *                         HLQ_backward_kernel.cu:533-537,561,587-591)
 *   hot_gemm_i8          CutlassSgemmNN_int4 / CutlassSgemmNN_int8 +
 *                        dequantize_cuda(_per_token)_kernel
 *                        (HLQ_backward_kernel.cu:181-280,309-384,386-450)
 *   hot_abc_forward      FLinearQ.setup_context (utils/quant_matmul.py:178-212)
 *   hot_linear_backward  backward_cuda (HLQ_backward_kernel.cu:457-737) with
 *                        the numerics of FLinearQ.backward, scheme gih_gwlr
 *                        (utils/quant_matmul.py:215-348)
 *   hot_*_batched        the same two on [B, T, C] tensors with the quantisers
 *                        vmapped over the batch (utils/quant_matmul.py:33-37,
 *                        102-106,118-122)
 *   hot_gx_lowrank       the g_x side of the schemes low_rank / gilr_gwh
 *                        (utils/quant_matmul.py:229-234,263-266,334-338)
 *   hot_gx_luq, hot_gw_luq   luq_quantizer on the g_y operand of either product
 *                        (utils/quant_matmul.py:58-83,250-253,307-314)
 *   hot_gemm_bf16        F.linear of the forward pass (utils/quant_matmul.py:173-176)
 */
#ifndef HOT_GFX950_H
#define HOT_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HOT_ABI_VERSION 4
#define HOT_API __attribute__((visibility("default")))

enum hot_status {
  HOT_OK = 0,
  HOT_ERR_INVALID = -1,     /* bad argument (null pointer, bad enum, bad size) */
  HOT_ERR_UNSUPPORTED = -2, /* shape or option outside what the kernels cover */
  HOT_ERR_WORKSPACE = -3,   /* workspace too small */
  HOT_ERR_HIP = -4          /* a HIP runtime call failed */
};

enum hot_dtype { HOT_F32 = 0, HOT_BF16 = 1, HOT_F16 = 2 };
/* HOT_ROUND_NEAREST: rint(x / fl32(s + 1e-11)), ties to even, IEEE division (int_quantizer_BWD,
 *   utils/quant_matmul.py:108-116).
 * HOT_ROUND_STOCH: floor|y| + 1 with probability frac|y|, y = x / fl32(s + 1e-11) (stoch_quantizer_BWD /
 *   norm_quantizer_BWD, :19-31, 86-100), from a counter-based generator instead of the reference's global
 *   one: element e draws the 16-bit integer r_e = halfword (e & 7) of the Philox-4x32-7 output for counter
 *   (e >> 3 lo, e >> 3 hi, stream, 0) under key (seed lo, seed hi), and the code is
 *   sign(x) min((trunc(fma(|x|, fl32(1 / d) 2^16, 0.5)) + r_e) >> 16, qmax): the expectation is y within
 *   2^-15 of a step.  The numbering of the elements is stated with every entry point. */
enum hot_rounding { HOT_ROUND_NEAREST = 0, HOT_ROUND_STOCH = 1 };
enum hot_scale_mode {
  HOT_SCALE_TENSOR = 0, /* one absmax step for the whole tensor */
  HOT_SCALE_ROW = 1,    /* one absmax step per row of the quantised matrix */
  HOT_SCALE_SAWB = 2    /* one step from clip = 12.1 rms - 12.2 mean|.| */
};

/* Counter-based RNG stream identifiers (Philox counter word 2). */
enum hot_rng_stream { HOT_STREAM_GX = 0, HOT_STREAM_GW = 1, HOT_STREAM_W = 2, HOT_STREAM_ACT = 3 };

#define HOT_HQ_WORKSPACE_BYTES 2048 /* per-tensor absmax of hot_hq_rowwise: 16 partial maxima, one per 128-byte line */
#define HOT_MAX_HLA_N 64        /* largest block with its rows inline in hot_config     */
#define HOT_MAX_HLA_BIG 8192    /* largest block at all (rows through hla_rows_big)     */

/* Options of the fused path; mirrors the fields FLinearQ reads from the
 * reference's module-global `args` (args.py:29-49), scheme gih_gwlr. */
typedef struct hot_config {
  int32_t n_o;      /* Hadamard block along O: a power of two, 1 .. 64            */
  int32_t hla_n;    /* HLA block along tokens: a power of two, 1 .. HOT_MAX_HLA_BIG */
  int32_t hla_r;    /* kept coefficients per block, 1..hla_n                      */
  int32_t hla_rows[HOT_MAX_HLA_N]; /* natural-order row of output coefficient k
                                      (blocks up to HOT_MAX_HLA_N)                */
  int32_t gx_bits, w_bits, gw_bits, act_bits;         /* 4 or 8                   */
  int32_t gx_round, w_round, gw_round, act_round;     /* hot_rounding             */
  int32_t gx_scale, w_scale, gw_scale, act_scale;     /* hot_scale_mode           */
  uint64_t seed;    /* stochastic-rounding key                                    */
  const int32_t* hla_rows_big; /* host, hla_r entries: the rows of blocks above
                                  HOT_MAX_HLA_N tokens (NULL otherwise); read
                                  during the call only.  Blocks of 128 tokens run
                                  in the same kernels as smaller ones; from 256 on
                                  they take a two-level transform through an fp32
                                  workspace (launches only: capturable)          */
  int32_t streams;  /* launch order of hot_linear_backward(_bias): 0 = the library's rule
                       (hot_backward_streams), 1 = every kernel on the caller's stream, 2 =
                       independent kernels also on the library's side stream (forked and joined by
                       events).  The results do not depend on it.                               */
  int32_t reserved; /* 0 */
} hot_config;

HOT_API const char* hot_last_error(void);
/* 1 or 2: the launch order hot_linear_backward takes for this shape (cfg->streams when it is 1 or 2).
 * Short calls, whose kernels take less time than the host needs for the event operations that fork
 * and join the side stream, run on one stream; long ones overlap their independent kernels. */
HOT_API int hot_backward_streams(int64_t L, int64_t O, int64_t I, const hot_config* cfg);
HOT_API int hot_abi_version(void);

/* Bytes of the leading dimension (row pitch) the library uses for a K-major
 * int8 code matrix with `k` codes per row: k rounded up to the GEMM K-tile. */
HOT_API int64_t hot_kpad(int64_t k);

/*
 * Block-Hadamard along the contiguous dimension + absmax step + quantise.
 *   in          device, [M, K] row-major, dtype
 *   n           Hadamard block, a power of two 1 .. 64; K % n == 0 and K % 8 == 0
 *   bits        4: codes_out is [M, K/2] bytes, element 2j in bits 3:0 of byte j
 *               8: codes_out is [M, K] int8
 *   scale_mode  HOT_SCALE_TENSOR -> scales_out[1]; HOT_SCALE_ROW -> scales_out[M]
 *   workspace   device, >= HOT_HQ_WORKSPACE_BYTES, 256-byte aligned (TENSOR mode only)
 */
HOT_API int hot_hq_rowwise(const void* in, int dtype, int64_t M, int64_t K, int n, int bits,
                   int rounding, uint64_t seed, uint32_t rng_stream, int scale_mode,
                   void* codes_out, float* scales_out, void* workspace,
                   size_t workspace_bytes, void* hip_stream);

/*
 * Hadamard low-rank projection along the row (token) dimension, quantise, and
 * store TRANSPOSED (K-major) for the int8 GEMM.
 *   in          device, [R, C] row-major, dtype; R % n == 0
 *   rows        host, r natural-order row indices in [0, n)
 *   codes_out   device, logical [C, (R/n)*r] codes; row pitch ld_out bytes;
 *               bytes beyond the logical row up to ld_out are written as zero
 *   scales_out  [1] (TENSOR, SAWB) or [C] (ROW)
 *   workspace   device, >= hot_hla_workspace_bytes(R, C, n, r)
 * Stochastic rounding numbers the kept coefficients of block b of channel c
 * in increasing natural-row order v = 0..r-1 and gives coefficient v the RNG
 * element index ((c * (R/n) + b) * rpad + v), rpad = r rounded up to 8.
 */
HOT_API int hot_hla_tokenwise(const void* in, int dtype, int64_t R, int64_t C, int n,
                      const int32_t* rows, int r, int bits, int rounding, uint64_t seed,
                      uint32_t rng_stream, int scale_mode, void* codes_out, int64_t ld_out,
                      float* scales_out, void* workspace, size_t workspace_bytes,
                      void* hip_stream);

/* Full block-Hadamard (all n rows kept) along the row dimension of W [O, I],
 * quantise, store as [I, O] codes (K-major).  Same conventions as above. */
HOT_API int hot_wq_colwise(const void* in, int dtype, int64_t O, int64_t I, int n, int bits,
                   int rounding, uint64_t seed, uint32_t rng_stream, int scale_mode,
                   void* codes_out, int64_t ld_out, float* scales_out, void* workspace,
                   size_t workspace_bytes, void* hip_stream);

/*
 * hot_hla_tokenwise without a workspace argument and without any allocation: for callers that
 * cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference, whose op allocates every intermediate per call
 * (HLQ_backward_kernel.cu:518-522,557-563).  The kernels' scratch (statistics words, per-channel
 * maxima, per-workgroup sums: about 1.5 MiB) is a fixed array in the library's device code; each GPU
 * the library runs on holds it until the process ends.  Limits: C <= HOT_STATIC_MAX_CHANNELS and
 * n <= 128 (larger blocks need a workspace as large as the input); anything beyond is refused with
 * HOT_ERR_UNSUPPORTED.  All calls on one GPU share the array: calls that overlap on one GPU (two
 * streams, two threads) race and must be serialised by the caller.  Same results as
 * hot_hla_tokenwise, bit for bit.
 */
#define HOT_STATIC_MAX_CHANNELS 16384
HOT_API int hot_hla_tokenwise_static(const void* in, int dtype, int64_t R, int64_t C, int n,
                             const int32_t* rows, int r, int bits, int rounding, uint64_t seed,
                             uint32_t rng_stream, int scale_mode, void* codes_out, int64_t ld_out,
                             float* scales_out, void* hip_stream);

HOT_API size_t hot_colwise_workspace_bytes(int64_t C);
/* Workspace of hot_hla_tokenwise for any block size: hot_colwise_workspace_bytes(C)
 * up to 128 tokens, plus an fp32 copy of the input above. */
HOT_API size_t hot_hla_workspace_bytes(int64_t R, int64_t C, int n, int r);

/*
 * out[M, N] = ((acc * scale_a[row or 0]) * scale_b[0]) * post_scale,
 * acc[M, N] (int32) = A[M, K] . B[N, K]^T on integer codes (MFMA int8).
 *   A, B        device, K-major codes, both `bits` wide (4: packed nibbles,
 *               8: int8); row pitches lda, ldb in BYTES, each >= the bytes of
 *               hot_kpad(K) codes, and the codes in [K, hot_kpad(K)) must be 0
 *   scale_a     device; [M] when a_per_row != 0, else [1]
 *   out         device, [M, N] row-major of out_dtype, pitch ldo ELEMENTS
 *   acc_out     device int32 [M, N] (pitch N) or NULL
 */
HOT_API int hot_gemm_i8(const void* A, int64_t lda, const void* B, int64_t ldb, int bits,
                int64_t M, int64_t N, int64_t K, const float* scale_a, int a_per_row,
                const float* scale_b, float post_scale, void* out, int out_dtype,
                int64_t ldo, int32_t* acc_out, void* hip_stream);

/*
 * out[M, N] = A[M, K] . B[N, K]^T (+ bias[N]) on bf16 operands with fp32 accumulation: the plain
 * linear layer of the forward pass, y = x W^T + b (utils/quant_matmul.py:173-176, F.linear), through
 * the data path of the integer kernels (a lane's 16 bytes are eight bf16 of K).
 *   A, B     device, bf16, K-major; row pitches lda, ldb in BYTES (multiples of 16, >= 2 K);
 *            K a multiple of 128
 *   bias     device, N elements of out_dtype, or NULL
 *   out      device, [M, N] row-major of out_dtype (HOT_BF16 or HOT_F32), pitch ldo ELEMENTS
 *   variant  HOT_GEMM_AUTO, HOT_GEMM_SLOT_128, HOT_GEMM_SLOT_256 or HOT_GEMM_SLOT_160X256
 * The sums are added in the kernel's own order: the result equals the vendor library's to fp32
 * rounding of a sum over K, not bit for bit.
 */
HOT_API int hot_gemm_bf16(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t M, int64_t N,
                  int64_t K, const void* bias, void* out, int out_dtype, int64_t ldo, int variant,
                  void* hip_stream);

/* Forward-side activation buffer: xq[I, hot_kpad(L')] = quant8(P x)^T, sx[1]. */
HOT_API size_t hot_abc_workspace_bytes(int64_t L, int64_t I, const hot_config* cfg);
HOT_API int hot_abc_forward(const void* x, int dtype, int64_t L, int64_t I, const hot_config* cfg,
                    void* xq_out, float* sx_out, void* workspace, size_t workspace_bytes,
                    void* hip_stream);

/*
 * The fused backward: g_x[L, I] and g_W[O, I] (both of out_dtype, dense).
 *   gy [L, O], w [O, I] of dtype; xq / sx as written by hot_abc_forward
 *   times4      host, NULL or 4 floats in the order of the reference op's time
 *               vector {fwht, quant, gemm, dequant} (HLQ_backward_kernel.cu:729-733):
 *               seconds spent in {the transform passes that only measure (statistics
 *               of g_y and W), the transform+quantise passes (g_y twice, W), both
 *               GEMMs, 0: dequantisation is the GEMMs' epilogue}; non-NULL makes
 *               the call synchronise the stream and run its kernels one after the
 *               other on `hip_stream`
 * Without timing, independent kernels of the call (the two W kernels, the row-wise
 * quantise pass of g_y and, for products too small to fill the chip, the g_x GEMM) run
 * on a side stream of the library (one per device, created on first use, default
 * priority) between events recorded on `hip_stream` and a wait on it, so they overlap
 * the token-wise g_y kernels and the g_W GEMM; everything is ordered after earlier
 * work on `hip_stream` and before later work on it.
 */
HOT_API size_t hot_backward_workspace_bytes(int64_t L, int64_t O, int64_t I, const hot_config* cfg);
HOT_API int hot_linear_backward(const void* gy, const void* w, int dtype, const void* xq,
                        const float* sx, int64_t L, int64_t O, int64_t I,
                        const hot_config* cfg, void* gx, void* gw, int out_dtype,
                        void* workspace, size_t workspace_bytes, float* times4,
                        void* hip_stream);

/*
 * hot_linear_backward (without stage timings) that also returns the bias gradient
 * gb[O] of out_dtype: the sum of g_y over the tokens, accumulated in fp32 in a fixed order
 * (within a token block in the butterfly order of the transform, whose coefficient 0 it
 * is; then block after block) and rounded once.  It costs no pass over g_y: the statistics
 * pass of the token-wise kernel already holds every block's sum.  The reference adds the
 * bias outside its autograd Function (utils/quant_matmul.py:419-420), so there the bias
 * gradient is autograd's own reduction of g_y; this entry point folds that reduction into
 * the backward of the layer.  Same workspace as hot_linear_backward.
 */
HOT_API int hot_linear_backward_bias(const void* gy, const void* w, int dtype, const void* xq,
                             const float* sx, int64_t L, int64_t O, int64_t I,
                             const hot_config* cfg, void* gx, void* gw, void* gb, int out_dtype,
                             void* workspace, size_t workspace_bytes, void* hip_stream);

/*
 * 3-D activations [B, T, C]: the reference vmaps its quantisers over the batch dimension, so every
 * sample has steps of its own, applies the token-wise transform inside each sample and sums the
 * per-sample weight gradients (utils/quant_matmul.py:33-37,102-106,118-122,288-290,322-324;
 * utils/hadamard_matmul.py:143-161).  These two entry points take the B samples as the rows
 * [b T, (b + 1) T) of the flattened tensors and do one call per layer:
 *   hot_abc_forward_batched      xq [I, B * kg] int8, kg = hot_kpad_group(T, cfg) (the codes of sample b
 *                                in bytes [b kg, (b + 1) kg) of every row, zero behind its T' codes),
 *                                sx [B]; cfg->hla_n must divide T and be at most 128
 *   hot_linear_backward_batched  g_x [B T, I], g_W [O, I] = sum over samples, each sample's integer
 *                                sums dequantised with its own steps and added in fp32
 *   hot_backward_batched_ranges  the order of that fp32 sum: the samples are cut into this many ranges
 *                                of ceil(B / ranges) consecutive samples (a function of the shape
 *                                alone); a range is summed in sample order, the range sums are added
 *                                in range order.  (The reference leaves the order to torch's sum over
 *                                the batch dimension.)  0 = bad arguments.
 * Per-tensor steps become per-sample steps, per-token steps stay per token, per-channel steps of the g_W
 * operand become per sample and channel.  Stochastic rounding numbers the elements as the flattened
 * calls do.  Everything runs on `hip_stream` in order.
 */
HOT_API int64_t hot_kpad_group(int64_t T, const hot_config* cfg);
HOT_API size_t hot_abc_batched_workspace_bytes(int64_t B, int64_t T, int64_t I, const hot_config* cfg);
HOT_API int hot_abc_forward_batched(const void* x, int dtype, int64_t B, int64_t T, int64_t I,
                            const hot_config* cfg, void* xq_out, float* sx_out, void* workspace,
                            size_t workspace_bytes, void* hip_stream);
HOT_API size_t hot_backward_batched_workspace_bytes(int64_t B, int64_t T, int64_t O, int64_t I,
                                            const hot_config* cfg);
HOT_API int hot_backward_batched_ranges(int64_t B, int64_t T, int64_t O, int64_t I, const hot_config* cfg);
HOT_API int hot_linear_backward_batched(const void* gy, const void* w, int dtype, const void* xq,
                                const float* sx, int64_t B, int64_t T, int64_t O, int64_t I,
                                const hot_config* cfg, void* gx, void* gw, int out_dtype,
                                void* workspace, size_t workspace_bytes, void* hip_stream);

/*
 * g_x of the schemes that project g_y to low rank along the TOKENS for that product
 * (utils/quant_matmul.py, transform_scheme "low_rank" and "gilr_gwh": :229-233 g_y <- P g_y,
 * :263-266 W untransformed, :288-290 the product and its two steps, :334-337 P^T (.) / n):
 *   g_x [L, I] = P^T ( q(P g_y) [L', O] . q(W) [O, I] ) s_g s_w / hla_n.
 * cfg->hla_n / hla_rows (hla_rows_big above 64) describe P: blocks up to 128 tokens in one pass,
 * 256 .. 8192 through the two-level path in both directions (fp32 intermediates in the workspace).
 * gx_bits / gx_round / gx_scale are the quantiser of P g_y: HOT_SCALE_TENSOR (one step; elements of
 * stochastic rounding numbered as hot_hla_tokenwise numbers them) or HOT_SCALE_ROW (one step per
 * coefficient row of [L', O], as norm_quantizer gives them; blocks up to 128 tokens; elements
 * numbered row-major).  w_bits (= gx_bits) / w_round / w_scale are the quantiser of W.  The g_W
 * side of those schemes is the g_W side of hot_linear_backward with the matching token-wise
 * selection (hot_hla_tokenwise + hot_gemm_i8).  Four to eight kernels on `hip_stream`, kept for
 * completeness of the reference's scheme list.
 */
HOT_API size_t hot_gx_lowrank_workspace_bytes(int64_t L, int64_t O, int64_t I, const hot_config* cfg);
HOT_API int hot_gx_lowrank(const void* gy, const void* w, int dtype, int64_t L, int64_t O, int64_t I,
                   const hot_config* cfg, void* gx, int out_dtype, void* workspace,
                   size_t workspace_bytes, void* hip_stream);

/*
 * g_x with the logarithmic unbiased quantiser on g_y (quantBWDGogi = "luq",
 * utils/quant_matmul.py:58-83,252-253): g_x = (luq(g_y blkdiag(H)) . q(blkdiag(H) W)) s_g s_w / n_o.
 * luq_quantizer_BWD: s = max(t) / 2^lev, lev = 2^(bits-1) - 1; magnitudes below s become s with
 * probability |t| / s, else 0; others 2^k s or 2^(k+1) s with the probabilities that keep the
 * expectation.  gx_bits = w_bits = 4.  The codes (0, +-2^j) are no uniform grid: they go through
 * the INT8 product as two planes (q = 16 a + b) against [16 w | w].  Element e of the row-major
 * transformed g_y draws the uniforms 2 e and 2 e + 1 of Philox stream 4 under cfg->seed
 * (cfg->gx_round and gx_scale are not read).
 * Stated deviation: the two planes carry codes up to +-2^10, and larger ones saturate there.  The
 * reference's step comes from the maximum, not from the largest magnitude (:60-61), so a negative
 * element of at least eight times the positive maximum of the transformed tensor would take a larger
 * code in the reference (which multiplies in floating point); here it is held at -2^10 s.
 */
HOT_API size_t hot_gx_luq_workspace_bytes(int64_t L, int64_t O, int64_t I, const hot_config* cfg);
HOT_API int hot_gx_luq(const void* gy, const void* w, int dtype, int64_t L, int64_t O, int64_t I,
               const hot_config* cfg, void* gx, int out_dtype, void* workspace,
               size_t workspace_bytes, void* hip_stream);

/*
 * g_W with the logarithmic quantiser on the projected g_y (quantBWDGogw = "luq", or luq_quantizer
 * picked for a layer's g_W under quantAuto, utils/quant_matmul.py:296-301,307-314,322-324):
 * g_W[O, I] = (luq((P g_y)^T) . xq^T) s sx / hla_n, xq / sx as written by hot_abc_forward
 * ([I, hot_kpad(L')] INT8 codes, one step).  gw_bits = 4, token blocks up to 128.  Element
 * e = o K8 + k of the projected tensor [O, L'] (K8 = L' rounded up to 8) draws the uniforms 2 e and
 * 2 e + 1 of Philox stream 5 under cfg->seed; codes saturate at +-2^10 as in hot_gx_luq.
 */
HOT_API size_t hot_gw_luq_workspace_bytes(int64_t L, int64_t O, int64_t I, const hot_config* cfg);
HOT_API int hot_gw_luq(const void* gy, int dtype, const void* xq, const float* sx, int64_t L, int64_t O,
               int64_t I, const hot_config* cfg, void* gw, int out_dtype, void* workspace,
               size_t workspace_bytes, void* hip_stream);

/*
 * Number of K ranges into which the GEMMs inside hot_linear_backward cut a product of
 * M x N outputs over K codes of `bits` bits (1 = one kernel; more = a kernel per range
 * writing int32 partial tiles to the workspace, then a reduce kernel).  Products with
 * few (below 96) 128 x 128 output tiles and a long K are cut so that the whole chip takes
 * part.  hot_gemm_i8 itself has no workspace and never splits.  No counterpart in the
 * reference (its CUTLASS GEMMs run without split-K, HLQ_backward_kernel.cu:236-250).
 */
HOT_API int hot_gemm_splits(int64_t M, int64_t N, int64_t K, int bits);

/*
 * Kernel variants of the integer GEMM.  hot_gemm_i8 and the GEMMs inside hot_linear_backward pick
 * one per product (hot_gemm_plan tells which); hot_gemm_i8_variant runs a named one, so that tests
 * and measurements can cover every kernel whatever the rule picks.  The reference has no
 * counterpart: its two CUTLASS instantiations are fixed at compile time
 * (cuda_measure/HLQ_backward_kernel.cu:181-280,309-384).
 */
enum hot_gemm_variant {
  HOT_GEMM_AUTO = 0,           /* let the library choose                                        */
  HOT_GEMM_DMA_128_S3 = 1,     /* 128 x 128 tiles, operands HBM -> LDS directly, ring of 3 stages */
  HOT_GEMM_DMA_128_S4 = 2,     /* the same with 4 stages                                        */
  HOT_GEMM_DMA_256_S4 = 3,     /* 256 x 256 tiles, ring of 4 stages                             */
  HOT_GEMM_REG_128 = 4,        /* 128 x 128 tiles staged through registers (operands >= 4 GiB)  */
  HOT_GEMM_DMA_128_SPLITK = 5, /* 128 x 128 tiles, K cut into ranges + reduce kernel; needs a
                                  workspace of hot_gemm_workspace_bytes                         */
  /* Slot-scheduled kernels: the K loop laid out by hand, one MFMA per slot with the fragment reads,
     the INT4 expansion and the DMA issue in its shadow; stages of 128 bytes per row (whole cache
     lines), so they take rows (K codes rounded up to 128, times bits / 8) of a multiple of 128 bytes */
  HOT_GEMM_SLOT_256 = 6,       /* 256 x 256 tiles, two stages                                   */
  HOT_GEMM_SLOT_128 = 7,       /* 128 x 128 tiles, four stages, one workgroup per CU            */
  HOT_GEMM_SLOT_160X256 = 8,   /* 160 x 256 tiles (four waves side by side), two stages         */
  HOT_GEMM_SLOT_96X128 = 9,    /* 96 x 128 tiles (four waves side by side), four stages, INT8   */
  HOT_GEMM_SLOT_64X128 = 10,   /* 64 x 128 tiles (four waves side by side), four stages, INT8   */
  HOT_GEMM_SLOT_32X128 = 11,   /* 32 x 128 tiles (four waves side by side), four stages, INT8   */
  HOT_GEMM_VARIANTS = 12
};
/* The variant hot_gemm_i8 (workspace_bytes = 0) or a GEMM inside hot_linear_backward
 * (workspace_bytes = what the call can spare) runs for this product; lda, ldb in bytes. */
HOT_API int hot_gemm_plan(int64_t M, int64_t N, int64_t K, int bits, int64_t lda, int64_t ldb,
                          size_t workspace_bytes);
/* Workspace with which the split-K variant runs for this product (0: it does not apply). */
HOT_API size_t hot_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits);
/* hot_gemm_i8 with the kernel named by `variant` (HOT_GEMM_AUTO: the library's choice given the
 * workspace); `workspace` may be NULL for the variants that need none.  A variant that does not
 * apply to the product (split-K without a long K, a DMA kernel on operands of 4 GiB or more) is
 * refused with HOT_ERR_UNSUPPORTED. */
HOT_API int hot_gemm_i8_variant(const void* A, int64_t lda, const void* B, int64_t ldb, int bits,
                        int64_t M, int64_t N, int64_t K, const float* scale_a, int a_per_row,
                        const float* scale_b, float post_scale, void* out, int out_dtype,
                        int64_t ldo, int32_t* acc_out, int variant, void* workspace,
                        size_t workspace_bytes, void* hip_stream);

/*
 * hot_linear_backward with a HIP event after every kernel group; synchronises
 * the stream.  times8 (host) receives the seconds of
 *   [0] clearing the statistics          [1] token-wise statistics pass over g_y
 *   [2] token-wise quantise pass (g_y)   [3] row-wise quantise pass(es) (g_y)
 *   [4] statistics pass over W           [5] quantise pass over W
 *   [6] g_x GEMM                         [7] g_W GEMM (both launches when split)
 * The reference has no counterpart beyond the four clock() stage timers its op
 * returns (cuda_measure/HLQ_backward_kernel.cu:717-733); this is the
 * measurement hook of bench.py.
 */
HOT_API int hot_linear_backward_kernels(const void* gy, const void* w, int dtype, const void* xq,
                                const float* sx, int64_t L, int64_t O, int64_t I,
                                const hot_config* cfg, void* gx, void* gw, int out_dtype,
                                void* workspace, size_t workspace_bytes, float* times8,
                                void* hip_stream);

/*
 * What this box can do at most, from two plain kernels: a device-to-device copy (copy_gbs: bytes read
 * + bytes written per second, in GB/s) and a loop of independent INT8 MFMAs, one wave per SIMD
 * (mfma_tops, in TOP/s).  bench.py reports them beside the published peaks.  `scratch`: device
 * memory, at least 64 MiB (the copy moves its first half onto its second).  Synchronises the stream.
 * No counterpart in the reference.
 */
HOT_API int hot_measure_ceilings(void* scratch, size_t scratch_bytes, float* copy_gbs, float* mfma_tops,
                         void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* HOT_GFX950_H */
