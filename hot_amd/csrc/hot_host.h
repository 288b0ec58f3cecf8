// Host-side plumbing shared by the translation units of libhot_gfx950:
// error reporting and the internal (C++) entry points behind the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/hot_gfx950.h"

namespace hot {

// Records the message for hot_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// hipGetLastError() after a launch -> HOT_OK or HOT_ERR_HIP.
int check_launch(const char* what);
int check_hip(hipError_t e, const char* what);

inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

constexpr int64_t GEMM_KTILE = 128;  // codes per K-tile of the int8 GEMM
constexpr int COL_MAX_N = 128;       // largest token block one thread transforms in registers

// A per-tensor absmax is collected in STAT_SLOTS partial maxima, one per 128-byte line, and the
// consumers take the maximum of the slots: thousands of workgroups updating ONE address queue up
// behind each other at the memory side (measured: 10 us of a 29 us statistics pass).
constexpr int STAT_SLOTS = 16;
constexpr int STAT_SLOT_STRIDE = 32;                                   // floats between slots
constexpr size_t STAT_SLOT_BYTES = (size_t)STAT_SLOTS * STAT_SLOT_STRIDE * 4;   // 2048

int hq_rowwise_impl(const void* in, int dtype, int64_t M, int64_t K, int n, int bits, int rounding,
                    uint64_t seed, uint32_t rng_stream, int scale_mode, void* codes_out, int64_t ld_codes,
                    float* scales_out, void* workspace, size_t workspace_bytes, hipStream_t st,
                    bool absmax_ready = false, int64_t group_rows = 0, float* group_steps = nullptr);
// group_rows > 0 (per-tensor steps only): every run of group_rows rows is a sample with a step of its
// own; scales_out then holds M entries (the step of each row's sample, the form the GEMM epilogue
// reads), group_steps (may be null) the M / group_rows steps, and the workspace 128 bytes per sample.

// Logarithmic quantiser of the row-wise transformed tensor (luq_quantizer_BWD): codes 0 / +-2^j split as
// 16 a + b into two planes of kp bytes per row ([M, 2 kp]), one step; the workspace holds STAT_SLOT_BYTES.
int hq_luq_impl(const void* in, int dtype, int64_t M, int64_t K, int n, int bits, uint64_t seed, void* codes_out,
                int64_t kp, float* scale_out, void* workspace, size_t workspace_bytes, hipStream_t st,
                uint32_t rng_stream = 4);
// RNG streams of the logarithmic quantiser: its operand of the g_x product, of the g_W product
constexpr uint32_t HOT_STREAM_LUQ = 4, HOT_STREAM_LUQ_GW = 5;
// Unquantised token-wise projection, transposed: out[c][blk r + k] = (P in)[blk r + k][c] in fp32, ld
// floats per channel (the tail [NB r, ld) cleared); or row-major: out[blk r + k][c], ld floats per
// coefficient row.  Blocks up to 128 tokens.
int hla_project_impl(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows, int r, float* out,
                     int64_t ld, hipStream_t st, bool rowmajor = false);
// out = ((float(16 acc_a + acc_b) * s_a[0]) * s_b[0]) * post on [M, N] int32 sums
int luq_combine_impl(const int32_t* acc_a, const int32_t* acc_b, int64_t M, int64_t N, const float* s_a, const float* s_b,
                     float post, void* out, int out_dtype, hipStream_t st);
// [rows, 2 kp] = [16 w | w] from INT8-stored codes w [rows, kp] with |w| <= 8
int luq_pair_impl(const void* qw, int64_t rows, int64_t kp, void* out, hipStream_t st);

int colwise_quant_impl(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows, int r,
                       int bits, int rounding, uint64_t seed, uint32_t rng_stream, int scale_mode,
                       void* codes_out, int64_t ld_out, int store4, float* scales_out, void* workspace,
                       size_t workspace_bytes, hipStream_t st, const char* who, float* row16_absmax_out = nullptr,
                       bool stats_cleared = false, hipEvent_t after_stats = nullptr, float* colsum_partial = nullptr,
                       int groups = 1, int64_t kpad_group = 0, bool rowmajor = false);
// rowmajor: codes stored untransposed, [NB r, C] with ld_out bytes per coefficient row (bytes past the C
// channels of a row are left alone: zero_pad_impl clears them), one step for the tensor.
void zero_pad_impl(void* codes, int64_t rows, int64_t row_bytes, int64_t ld, hipStream_t st);
// out[NB n, C] = (P^T t) * post for t [NB r, C] fp32: the kept coefficients go back to their natural rows of
// every block and the block is transformed again (H is symmetric); n up to 128.
int hla_expand_impl(const float* t, int64_t nb, int64_t C, int n, const int32_t* rows, int r, float post,
                    void* out, int out_dtype, hipStream_t st);
// The same for blocks of 256 .. 8192 tokens: two passes with the fp32 intermediate in the workspace.
int hla_expand_big_impl(const float* t, int64_t nb, int64_t C, int n, const int32_t* rows, int r, float post, void* out,
                        int out_dtype, void* workspace, size_t workspace_bytes, hipStream_t st);
size_t hla_expand_big_workspace_bytes_impl(int64_t nb, int64_t C, int n);
// With groups > 1 the R rows are `groups` samples of equal length, each quantised with steps of its own
// (scales_out: [groups], or [groups][C] with per-channel steps); the codes of sample g take the bytes
// [g * kpad_group, (g + 1) * kpad_group) of every output row, zero-filled behind the sample's codes.
size_t colwise_group_workspace_bytes_impl(int64_t C, int groups);
// Column sums of the input of a colwise_quant_impl call (the bias gradient when the input is g_y):
// with colsum_partial the call also writes colsum_strips_impl(...) rows of C partial sums (fp32; elem_bytes
// = size of an input element, on which the partition of the passes depends; one
// row per run of token blocks of its statistics pass, which holds the sum of every block as
// coefficient 0); colsum_finish_impl adds the rows in a fixed order and rounds once to the output type.
int64_t colsum_strips_impl(int64_t R, int64_t C, int n, int r, int store4, int mode, int elem_bytes);
int colsum_finish_impl(const float* partial, int64_t strips, int64_t C, void* out, int out_dtype, hipStream_t st);
size_t colwise_workspace_bytes_impl(int64_t C);
size_t colwise_stats_bytes_impl(int64_t C);  // leading part of the workspace that must be zero before the statistics pass

// Blocks of 256 .. 8192 tokens (two-level transform through an fp32 workspace); same contract as
// colwise_quant_impl without the packed-INT4 store.
int hla_big_impl(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows, int r, int bits,
                 int rounding, uint64_t seed, uint32_t rng_stream, int scale_mode, void* codes_out, int64_t ld_out,
                 float* scales_out, void* workspace, size_t workspace_bytes, hipStream_t st, const char* who,
                 hipEvent_t after_stats = nullptr, float* row16_absmax_out = nullptr, bool rowmajor = false,
                 int store4 = 0);
// rowmajor: the codes are stored untransposed, [NB r, C] with ld_out bytes per coefficient row (store4:
// two channels to a byte).
// row16_absmax_out (STAT_SLOTS partial maxima, zero before the call; C a multiple of 16, absmax steps):
// stage 1 also delivers the absmax of the row-wise 16-point Hadamard of the input.
size_t hla_big_workspace_bytes_impl(int64_t R, int64_t C, int n, int r);
// Workspace of a token-wise transform of [R, C] with blocks of n tokens and r kept rows, either path.
size_t hla_workspace_bytes_impl(int64_t R, int64_t C, int n, int r);

int gemm_i8_impl(const void* A, int64_t lda, const void* B, int64_t ldb, int bits, int64_t M, int64_t N,
                 int64_t K, const float* scale_a, int a_per_row, const float* scale_b, float post_scale,
                 void* out, int out_dtype, int64_t ldo, int32_t* acc_out, hipStream_t st, void* split_ws = nullptr,
                 size_t split_ws_bytes = 0, int variant = HOT_GEMM_AUTO);
int gemm_bf16_impl(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t M, int64_t N, int64_t K,
                   const void* bias, void* out, int out_dtype, int64_t ldo, hipStream_t st, int variant);
// The hot_gemm_variant that gemm_i8_impl picks for a product when `ws_bytes` of workspace come with it.
int gemm_plan_impl(int64_t M, int64_t N, int64_t K, int bits, int64_t lda, int64_t ldb, size_t ws_bytes);

// K groups with steps of their own: out = (sum over groups g, in the order below, of
// (float(A_g . B_g^T) * scale_a[g or g M + row]) * scale_b[g]) * post_scale.  The groups are cut into
// gemm_grouped_splits_impl(...) ranges of ceil(groups / ranges) consecutive groups; a range is summed in
// group order, the range sums are added in range order.  More than one range needs a workspace.
int gemm_i8_grouped_impl(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t M, int64_t N, int groups,
                         int64_t group_k, const float* scale_a, int a_per_row, const float* scale_b, float post_scale,
                         void* out, int out_dtype, int64_t ldo, void* workspace, size_t workspace_bytes, hipStream_t st);
int gemm_grouped_splits_impl(int64_t M, int64_t N, int groups, int64_t group_k);
size_t gemm_grouped_workspace_bytes_impl(int64_t M, int64_t N, int groups, int64_t group_k);

// Split-K plan of gemm_i8_impl for a problem: `splits` K ranges (1 = none) and the bytes of workspace
// that hold their partial accumulators (16-byte aligned; contents need no initialisation).
struct GemmSplit { int splits; size_t ws_bytes; };
GemmSplit gemm_split_plan(int64_t M, int64_t N, int64_t K, int bits);

}  // namespace hot
