// C ABI of libhot_gfx950 and the fused HOT linear backward.
//
// hot_linear_backward sequences the kernels of the path on one HIP stream in
// the stage order of the reference op backward_cuda
// (cuda_measure/HLQ_backward_kernel.cu:457-737: transform -> quantise ->
// low-rank -> GEMM x2 -> dequantise) with the numerics of FLinearQ.backward,
// scheme gih_gwlr (utils/quant_matmul.py:215-348).  hot_abc_forward is the
// forward-side activation buffer of FLinearQ.setup_context (:178-212).
#include <string.h>

#include <mutex>

#include "hot_device.h"
#include "hot_host.h"

namespace hot {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return HOT_OK;
  return fail(HOT_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int check_launch(const char* what) { return check_hip(hipGetLastError(), what); }

static const int32_t* cfg_rows(const hot_config* c) { return c->hla_n > HOT_MAX_HLA_N ? c->hla_rows_big : c->hla_rows; }

static int check_cfg(const hot_config* c, const char* who) {
  if (!c) return fail(HOT_ERR_INVALID, "%s: null config", who);
  if (c->n_o < 1 || c->n_o > 64 || (c->n_o & (c->n_o - 1))) return fail(HOT_ERR_UNSUPPORTED, "%s: n_o=%d (a power of two up to 64)", who, c->n_o);
  if (c->hla_n < 1 || c->hla_n > HOT_MAX_HLA_BIG || (c->hla_n & (c->hla_n - 1))) return fail(HOT_ERR_UNSUPPORTED, "%s: hla_n=%d (power of two up to %d)", who, c->hla_n, HOT_MAX_HLA_BIG);
  if (c->hla_n > HOT_MAX_HLA_N && !c->hla_rows_big) return fail(HOT_ERR_INVALID, "%s: hla_n=%d needs hla_rows_big", who, c->hla_n);
  if (c->hla_r < 1 || c->hla_r > c->hla_n) return fail(HOT_ERR_INVALID, "%s: hla_r=%d outside [1, %d]", who, c->hla_r, c->hla_n);
  if (c->streams < 0 || c->streams > 2) return fail(HOT_ERR_INVALID, "%s: streams=%d (0 = the library's rule, 1 or 2)", who, c->streams);
  const int bits[4] = {c->gx_bits, c->w_bits, c->gw_bits, c->act_bits};
  for (int i = 0; i < 4; ++i)
    if (bits[i] != 4 && bits[i] != 8) return fail(HOT_ERR_UNSUPPORTED, "%s: quantiser width %d (4 or 8)", who, bits[i]);
  return HOT_OK;
}

struct BwdLayout {
  int64_t ld_g, ld_w, ld_gp;                       // code pitches in bytes
  size_t off_hq, off_colw, off_colg, off_sg, off_sw, off_sgp, off_qg, off_qw, off_qgp, off_split, off_colsum, total;
  int64_t colsum_strips;                         // room for that many rows of partial column sums of g_y (bias gradient)
  size_t split_bytes;                            // split-K workspace shared by the two GEMMs
};

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

static BwdLayout bwd_layout(int64_t L, int64_t O, int64_t I, const hot_config* c) {
  BwdLayout b;
  const int64_t lp = (L / c->hla_n) * c->hla_r;
  b.ld_g = round_up(O, GEMM_KTILE) * c->gx_bits / 8;
  b.ld_w = round_up(O, GEMM_KTILE) * c->w_bits / 8;
  b.ld_gp = round_up(lp, GEMM_KTILE);
  size_t o = 0;
  b.off_hq = o;   o += STAT_SLOT_BYTES;
  b.off_colw = o; o += align256(colwise_workspace_bytes_impl(I));
  b.off_colg = o; o += align256(hla_workspace_bytes_impl(L, O, c->hla_n, c->hla_r));
  b.off_sg = o;   o += align256((size_t)L * 4);
  b.off_sw = o;   o += 256;
  b.off_sgp = o;  o += align256((size_t)O * 4);
  b.off_qg = o;   o += align256((size_t)L * b.ld_g);
  b.off_qw = o;   o += align256((size_t)I * b.ld_w);
  b.off_qgp = o;  o += align256((size_t)O * b.ld_gp);
  const GemmSplit px = gemm_split_plan(L, I, O, c->gx_bits), pw = gemm_split_plan(O, I, lp, 8);
  b.split_bytes = px.ws_bytes > pw.ws_bytes ? px.ws_bytes : pw.ws_bytes;
  b.off_split = o; o += align256(b.split_bytes);
  {  // the workspace query knows no input type: room for the larger partition of the two element sizes
    const int64_t s2 = colsum_strips_impl(L, O, c->hla_n, c->hla_r, 0, c->gw_scale, 2);
    const int64_t s4 = colsum_strips_impl(L, O, c->hla_n, c->hla_r, 0, c->gw_scale, 4);
    b.colsum_strips = s2 > s4 ? s2 : s4;
  }
  b.off_colsum = o; o += align256((size_t)b.colsum_strips * (size_t)O * 4);
  b.total = o;
  return b;
}

__global__ void clear3_kernel(uint32_t* p0, int n0, uint32_t* p1, int n1, uint32_t* p2, int n2) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n0) { p0[i] = 0u; return; }
  i -= n0;
  if (i < n1) { p1[i] = 0u; return; }
  i -= n1;
  if (i < n2) p2[i] = 0u;
}

// One stream or two.  Forking and joining the side stream costs the host three event record / wait
// pairs, about 60 us on top of the 23 us the ten launches take (measured); that is hidden only when
// the kernels of the call run longer than it.  Calls with little arithmetic (both products together
// below 30 GOP: ViT-B proj at 12608 tokens, 23 GOP, runs 75 us on one stream against 85 us with the
// side stream; qkv, 70 GOP, 123 against 108) keep everything on the caller's stream.
static int backward_streams(int64_t L, int64_t O, int64_t I, const hot_config* c) {
  if (c->streams == 1 || c->streams == 2) return c->streams;
  const double lp = (double)((L / c->hla_n) * c->hla_r);
  const double ops = 2.0 * (double)O * (double)I * ((double)L + lp);
  return ops < 3.0e10 ? 1 : 2;
}

static const int32_t* identity_rows() {
  struct Rows { int32_t v[HOT_MAX_HLA_N]; Rows() { for (int i = 0; i < HOT_MAX_HLA_N; ++i) v[i] = i; } };
  static const Rows rows;   // initialised once, thread-safe
  return rows.v;
}

}  // namespace hot

using namespace hot;

extern "C" {

const char* hot_last_error(void) { return g_err; }
int hot_abi_version(void) { return HOT_ABI_VERSION; }
int hot_backward_streams(int64_t L, int64_t O, int64_t I, const hot_config* cfg) {
  if (check_cfg(cfg, "hot_backward_streams") || L <= 0 || O <= 0 || I <= 0) return 0;
  return backward_streams(L, O, I, cfg);
}
int64_t hot_kpad(int64_t k) { return round_up(k, GEMM_KTILE); }

int hot_gemm_splits(int64_t M, int64_t N, int64_t K, int bits) {
  if (bits != 4 && bits != 8) return 1;
  const GemmSplit sp = gemm_split_plan(M, N, K, bits);
  const int64_t pitch = round_up(K, GEMM_KTILE) * bits / 8;
  return gemm_plan_impl(M, N, K, bits, pitch, pitch, sp.ws_bytes) == HOT_GEMM_DMA_128_SPLITK ? sp.splits : 1;
}

int hot_hq_rowwise(const void* in, int dtype, int64_t M, int64_t K, int n, int bits, int rounding,
                   uint64_t seed, uint32_t rng_stream, int scale_mode, void* codes_out, float* scales_out,
                   void* workspace, size_t workspace_bytes, void* hip_stream) {
  const int64_t ld = (bits == 4 || bits == 8) ? K * bits / 8 : 0;
  return hq_rowwise_impl(in, dtype, M, K, n, bits, rounding, seed, rng_stream, scale_mode, codes_out, ld,
                         scales_out, workspace, workspace_bytes, (hipStream_t)hip_stream);
}

size_t hot_colwise_workspace_bytes(int64_t C) { return colwise_workspace_bytes_impl(C > 0 ? C : 0); }

size_t hot_hla_workspace_bytes(int64_t R, int64_t C, int n, int r) {
  if (R <= 0 || C <= 0 || n < 1 || r < 1) return 0;
  return hla_workspace_bytes_impl(R, C, n, r);
}

int hot_hla_tokenwise(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows, int r,
                      int bits, int rounding, uint64_t seed, uint32_t rng_stream, int scale_mode,
                      void* codes_out, int64_t ld_out, float* scales_out, void* workspace,
                      size_t workspace_bytes, void* hip_stream) {
  return colwise_quant_impl(in, dtype, R, C, n, rows, r, bits, rounding, seed, rng_stream, scale_mode,
                            codes_out, ld_out, /*store4=*/0, scales_out, workspace, workspace_bytes,
                            (hipStream_t)hip_stream, "hot_hla_tokenwise");
}

int hot_wq_colwise(const void* in, int dtype, int64_t O, int64_t I, int n, int bits, int rounding,
                   uint64_t seed, uint32_t rng_stream, int scale_mode, void* codes_out, int64_t ld_out,
                   float* scales_out, void* workspace, size_t workspace_bytes, void* hip_stream) {
  if (n != 16 && n != 32 && n != 64) return fail(HOT_ERR_UNSUPPORTED, "hot_wq_colwise: Hadamard block %d (16, 32 or 64)", n);
  return colwise_quant_impl(in, dtype, O, I, n, identity_rows(), n, bits, rounding, seed, rng_stream, scale_mode,
                            codes_out, ld_out, /*store4=*/bits == 4, scales_out, workspace, workspace_bytes,
                            (hipStream_t)hip_stream, "hot_wq_colwise");
}

int hot_gemm_i8(const void* A, int64_t lda, const void* B, int64_t ldb, int bits, int64_t M, int64_t N,
                int64_t K, const float* scale_a, int a_per_row, const float* scale_b, float post_scale,
                void* out, int out_dtype, int64_t ldo, int32_t* acc_out, void* hip_stream) {
  return gemm_i8_impl(A, lda, B, ldb, bits, M, N, K, scale_a, a_per_row, scale_b, post_scale, out, out_dtype,
                      ldo, acc_out, (hipStream_t)hip_stream);
}

int hot_gemm_bf16(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t M, int64_t N, int64_t K,
                  const void* bias, void* out, int out_dtype, int64_t ldo, int variant, void* hip_stream) {
  return gemm_bf16_impl(A, lda, B, ldb, M, N, K, bias, out, out_dtype, ldo, (hipStream_t)hip_stream, variant);
}

int hot_gemm_plan(int64_t M, int64_t N, int64_t K, int bits, int64_t lda, int64_t ldb, size_t workspace_bytes) {
  return gemm_plan_impl(M, N, K, bits, lda, ldb, workspace_bytes);
}

size_t hot_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits) {
  if (bits != 4 && bits != 8) return 0;
  return gemm_split_plan(M, N, K, bits).ws_bytes;
}

int hot_gemm_i8_variant(const void* A, int64_t lda, const void* B, int64_t ldb, int bits, int64_t M, int64_t N,
                        int64_t K, const float* scale_a, int a_per_row, const float* scale_b, float post_scale,
                        void* out, int out_dtype, int64_t ldo, int32_t* acc_out, int variant, void* workspace,
                        size_t workspace_bytes, void* hip_stream) {
  return gemm_i8_impl(A, lda, B, ldb, bits, M, N, K, scale_a, a_per_row, scale_b, post_scale, out, out_dtype,
                      ldo, acc_out, (hipStream_t)hip_stream, workspace, workspace_bytes, variant);
}

size_t hot_abc_workspace_bytes(int64_t L, int64_t I, const hot_config* cfg) {
  if (!cfg || L <= 0 || I <= 0) return colwise_workspace_bytes_impl(I > 0 ? I : 0);
  return hla_workspace_bytes_impl(L, I, cfg->hla_n, cfg->hla_r);
}

int hot_abc_forward(const void* x, int dtype, int64_t L, int64_t I, const hot_config* cfg, void* xq_out,
                    float* sx_out, void* workspace, size_t workspace_bytes, void* hip_stream) {
  if (int e = check_cfg(cfg, "hot_abc_forward")) return e;
  if (L <= 0 || I <= 0 || L % cfg->hla_n) return fail(HOT_ERR_INVALID, "hot_abc_forward: L=%lld must be a positive multiple of hla_n=%d", (long long)L, cfg->hla_n);
  if (cfg->act_scale == HOT_SCALE_ROW) return fail(HOT_ERR_UNSUPPORTED, "hot_abc_forward: the activation buffer uses one step per tensor");
  const int64_t lp = (L / cfg->hla_n) * cfg->hla_r;
  return colwise_quant_impl(x, dtype, L, I, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, cfg->act_bits, cfg->act_round,
                            cfg->seed, HOT_STREAM_ACT, cfg->act_scale, xq_out, round_up(lp, GEMM_KTILE), 0,
                            sx_out, workspace, workspace_bytes, (hipStream_t)hip_stream, "hot_abc_forward");
}

size_t hot_backward_workspace_bytes(int64_t L, int64_t O, int64_t I, const hot_config* cfg) {
  if (check_cfg(cfg, "hot_backward_workspace_bytes") || L <= 0 || O <= 0 || I <= 0) return 0;
  return bwd_layout(L, O, I, cfg).total;
}

// Slots of the per-kernel timing of one backward (hot_linear_backward_kernels).
enum {
  K_CLEAR = 0,      // statistics cleared
  K_GY_STATS = 1,   // token-wise statistics pass over g_y (also the row-wise absmax when fused)
  K_GY_HLA = 2,     // token-wise quantise pass over g_y  -> g_W operand
  K_GY_HQ = 3,      // row-wise pass(es) over g_y          -> g_x operand
  K_W_STATS = 4,    // statistics pass over W
  K_W_QUANT = 5,    // quantise pass over W
  K_GEMM_GX = 6,
  K_GEMM_GW = 7,
  K_COUNT = 8
};

// The two W kernels are small (a few MB) and cannot fill the chip; they run on a side stream beside
// the g_y kernels.  One side stream and three events per device, created on first use (default
// priority) and kept for the life of the process; a mutex keeps the fork / join of one call together.
struct SideLane {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, fork2 = nullptr, join = nullptr;
  bool tried = false, ok = false;
};
static std::mutex g_side_mutex;
static SideLane g_side[64];

static SideLane* side_lane_locked() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  SideLane& s = g_side[dev];
  if (!s.tried) {
    s.tried = true;
    s.ok = hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) == hipSuccess &&
           hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) == hipSuccess &&
           hipEventCreateWithFlags(&s.fork2, hipEventDisableTiming) == hipSuccess &&
           hipEventCreateWithFlags(&s.join, hipEventDisableTiming) == hipSuccess;
    if (!s.ok) (void)hipGetLastError();
  }
  return s.ok ? &s : nullptr;
}

static int run_backward(const void* gy, const void* w, int dtype, const void* xq, const float* sx, int64_t L,
                        int64_t O, int64_t I, const hot_config* cfg, void* gx, void* gw, int out_dtype,
                        void* workspace, size_t workspace_bytes, hipEvent_t* ev /* K_COUNT + 1 or null */,
                        int* slot_of /* K_COUNT: kernel group measured by event pair i, i + 1 */, hipStream_t st,
                        void* gb = nullptr /* [O] of out_dtype: column sums of g_y, or null */) {
  const char* who = "hot_linear_backward";
  if (int e = check_cfg(cfg, who)) return e;
  if (!gy || !w || !xq || !sx || !gx || !gw) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (L <= 0 || O <= 0 || I <= 0) return fail(HOT_ERR_INVALID, "%s: bad shape L=%lld O=%lld I=%lld", who, (long long)L, (long long)O, (long long)I);
  if (O % cfg->n_o) return fail(HOT_ERR_INVALID, "%s: O=%lld is not a multiple of n_o=%d", who, (long long)O, cfg->n_o);
  if (L % cfg->hla_n) return fail(HOT_ERR_INVALID, "%s: L=%lld is not a multiple of hla_n=%d", who, (long long)L, cfg->hla_n);
  if (cfg->gx_bits != cfg->w_bits) return fail(HOT_ERR_UNSUPPORTED, "%s: gx_bits (%d) and w_bits (%d) must match", who, cfg->gx_bits, cfg->w_bits);
  if (cfg->gx_scale == HOT_SCALE_SAWB) return fail(HOT_ERR_UNSUPPORTED, "%s: SAWB applies to W and x only", who);
  if (cfg->w_scale == HOT_SCALE_ROW) return fail(HOT_ERR_UNSUPPORTED, "%s: W uses one step per tensor", who);
  if (cfg->gw_scale == HOT_SCALE_SAWB) return fail(HOT_ERR_UNSUPPORTED, "%s: SAWB applies to W and x only", who);
  // limits of the stages, checked here so that nothing has been launched when one of them refuses
  if (O % 8 || I % 8) return fail(HOT_ERR_UNSUPPORTED, "%s: O=%lld and I=%lld must be multiples of 8", who, (long long)O, (long long)I);
  if (O * I * 4 >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "%s: W of %lld x %lld elements exceeds the 32-bit offsets of the loader", who, (long long)O, (long long)I);
  if (cfg->hla_n <= COL_MAX_N && L * O * 4 >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "%s: g_y of %lld x %lld elements exceeds the 32-bit offsets of the loader", who, (long long)L, (long long)O);
  if (L >= (1ll << 31)) return fail(HOT_ERR_UNSUPPORTED, "%s: L too large", who);
  if (((uintptr_t)gy & 15) || ((uintptr_t)w & 15) || ((uintptr_t)xq & 15)) return fail(HOT_ERR_INVALID, "%s: gy, w and xq must be 16-byte aligned", who);
  const BwdLayout b = bwd_layout(L, O, I, cfg);
  if (!workspace || workspace_bytes < b.total) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, b.total, workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  uint8_t* ws = (uint8_t*)workspace;
  float* sg = (float*)(ws + b.off_sg);
  float* sw = (float*)(ws + b.off_sw);
  float* sgp = (float*)(ws + b.off_sgp);
  const int64_t lp = (L / cfg->hla_n) * cfg->hla_r;
  // timing: event i + 1 is recorded after the i-th kernel group of the launch order; slot_of[i] names it
  int seq = 0;
  auto mark = [&](int slot) {
    if (!ev) return;
    slot_of[seq] = slot;
    (void)hipEventRecord(ev[++seq], st);
  };
  // event to record between the two kernels of a token-wise call (statistics pass, quantise pass)
  auto mid = [&](int slot) -> hipEvent_t {
    if (!ev) return nullptr;
    slot_of[seq] = slot;
    return ev[++seq];
  };
  if (ev) (void)hipEventRecord(ev[0], st);
  // one launch zeroes every statistic of the call (absmax slots, per-channel maxima)
  {
    const int n0 = (int)(STAT_SLOT_BYTES / 4), n1 = (int)(colwise_stats_bytes_impl(I) / 4), n2 = (int)(colwise_stats_bytes_impl(O) / 4);
    const int total = n0 + n1 + n2;
    hipLaunchKernelGGL(clear3_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                       (uint32_t*)(ws + b.off_hq), n0, (uint32_t*)(ws + b.off_colw), n1, (uint32_t*)(ws + b.off_colg), n2);
  }
  mark(K_CLEAR);
  // W: Hadamard along O + quantise, stored [I, O]
  auto quantise_w = [&](hipStream_t s2) {
    return colwise_quant_impl(w, dtype, O, I, cfg->n_o, identity_rows(), cfg->n_o, cfg->w_bits, cfg->w_round, cfg->seed,
                              HOT_STREAM_W, cfg->w_scale, ws + b.off_qw, b.ld_w, cfg->w_bits == 4, sw,
                              ws + b.off_colw, colwise_workspace_bytes_impl(I), s2, who, nullptr, /*stats_cleared=*/true,
                              mid(K_W_STATS));
  };
  // Without per-kernel timing, independent kernels overlap on the side stream: first the W kernels
  // beside the g_y statistics.
  std::unique_lock<std::mutex> side_guard(g_side_mutex, std::defer_lock);
  SideLane* side = nullptr;
  if (!ev && backward_streams(L, O, I, cfg) == 2) {
    side_guard.lock();
    side = side_lane_locked();
    if (!side) side_guard.unlock();
  }
  // Once the side stream has been forked, every way out of this function joins it again: the
  // caller's stream waits for what the side stream was given, also when a later stage refuses, so
  // that no kernel of the call still runs (on the workspace) behind work the caller queues next,
  // and a capture of the caller's stream is never left with an unjoined branch.
  struct SideJoin {
    SideLane* side = nullptr;
    hipStream_t st = nullptr;
    bool forked = false, joined = false;
    ~SideJoin() {
      if (!forked || joined) return;
      if (hipEventRecord(side->join, side->stream) == hipSuccess) (void)hipStreamWaitEvent(st, side->join, 0);
    }
  } side_join;
  int rc = HOT_OK;
  if (side) {
    rc = check_hip(hipEventRecord(side->fork, st), "hipEventRecord");
    if (!rc) rc = check_hip(hipStreamWaitEvent(side->stream, side->fork, 0), "hipStreamWaitEvent");
    if (rc) return rc;
    side_join.side = side; side_join.st = st; side_join.forked = true;
    rc = quantise_w(side->stream);
    if (rc) return rc;
  }
  // g_y: HLA along tokens + quantise, transposed (g_W operand); Hadamard along O + quantise (g_x
  // operand).  With one step per tensor both quantisers need the absmax of their transform first:
  // the statistics pass of the token-wise kernel delivers both from a single read of g_y.
  const bool fuse = cfg->gx_scale == HOT_SCALE_TENSOR && cfg->n_o == 16 && O % 16 == 0 && cfg->gw_scale != HOT_SCALE_SAWB;
  // Side stream, beside the g_W GEMM on the main stream: always the row-wise quantise pass of g_y (a
  // streaming kernel next to a matrix kernel); the g_x GEMM too when the g_W GEMM has fewer tiles
  // than the chip has CUs and cannot fill it alone (two large GEMMs only get in each other's way).
  const bool hq_aside = side != nullptr;
  const bool gx_aside = side != nullptr && ((O + 127) / 128) * ((I + 127) / 128) < 256;
  rc = colwise_quant_impl(gy, dtype, L, O, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, cfg->gw_bits, cfg->gw_round,
                          cfg->seed, HOT_STREAM_GW, cfg->gw_scale, ws + b.off_qgp, b.ld_gp, 0, sgp,
                          ws + b.off_colg, hla_workspace_bytes_impl(L, O, cfg->hla_n, cfg->hla_r), st, who,
                          fuse ? (float*)(ws + b.off_hq) : nullptr, /*stats_cleared=*/true,
                          hq_aside ? side->fork2 : mid(K_GY_STATS), gb ? (float*)(ws + b.off_colsum) : nullptr);
  if (rc) return rc;
  // bias gradient: the partial column sums of the statistics pass, added up by a small kernel that
  // rides on the side stream behind the row-wise quantise pass, beside the large kernels of the main
  // stream (here, in order, when there is no side stream)
  auto finish_bias = [&](hipStream_t s2) {
    if (!gb) return (int)HOT_OK;
    const int64_t strips = colsum_strips_impl(L, O, cfg->hla_n, cfg->hla_r, 0, cfg->gw_scale, dtype == HOT_F32 ? 4 : 2);
    return colsum_finish_impl((const float*)(ws + b.off_colsum), strips, O, gb, out_dtype, s2);
  };
  if (!side && (rc = finish_bias(st))) return rc;
  mark(K_GY_HLA);
  // g_x operand of g_y on the side stream: a streaming kernel beside the g_W GEMM
  auto quantise_gy_rows = [&](hipStream_t s2) {
    return hq_rowwise_impl(gy, dtype, L, O, cfg->n_o, cfg->gx_bits, cfg->gx_round, cfg->seed, HOT_STREAM_GX,
                           cfg->gx_scale, ws + b.off_qg, b.ld_g, sg, ws + b.off_hq, STAT_SLOT_BYTES, s2, fuse);
  };
  auto gemm_gx = [&](hipStream_t s2) {
    // g_x = (qG . qW^T) sG sW / n_o   (never split here: the split workspace belongs to the g_W GEMM)
    return gemm_i8_impl(ws + b.off_qg, b.ld_g, ws + b.off_qw, b.ld_w, cfg->gx_bits, L, I, O, sg,
                        cfg->gx_scale == HOT_SCALE_ROW, sw, 1.0f / (float)cfg->n_o, gx, out_dtype, I, nullptr, s2,
                        s2 == st && b.split_bytes ? ws + b.off_split : nullptr, s2 == st ? b.split_bytes : 0);
  };
  if (hq_aside) {
    // The statistics pass on the main stream feeds the row-wise quantiser only when it delivers the
    // fused absmax; with per-token steps (or an absmax pass of its own) the row-wise kernel starts
    // at once, beside the statistics pass.  The partial column sums always come from that pass.
    if (fuse) rc = check_hip(hipStreamWaitEvent(side->stream, side->fork2, 0), "hipStreamWaitEvent");
    if (!rc) rc = quantise_gy_rows(side->stream);
    if (!rc && gb && !fuse) rc = check_hip(hipStreamWaitEvent(side->stream, side->fork2, 0), "hipStreamWaitEvent");
    if (!rc) rc = finish_bias(side->stream);
    if (!rc && gx_aside) rc = gemm_gx(side->stream);
    if (rc) return rc;
  }
  if (side) {
    rc = check_hip(hipEventRecord(side->join, side->stream), "hipEventRecord");
    if (rc) return rc;
  }
  // g_W = (qGp . xq^T) sGp sx / hla_n, right after the kernel that wrote its large operand
  rc = gemm_i8_impl(ws + b.off_qgp, b.ld_gp, xq, b.ld_gp, 8, O, I, lp, sgp, cfg->gw_scale == HOT_SCALE_ROW, sx,
                    1.0f / (float)cfg->hla_n, gw, out_dtype, I, nullptr, st,
                    b.split_bytes ? ws + b.off_split : nullptr, b.split_bytes);
  if (rc) return rc;
  mark(K_GEMM_GW);
  if (!hq_aside) {
    rc = quantise_gy_rows(st);
    if (rc) return rc;
    mark(K_GY_HQ);
  }
  if (side) {
    rc = check_hip(hipStreamWaitEvent(st, side->join, 0), "hipStreamWaitEvent");
    if (rc) return rc;
    side_join.joined = true;
  } else {
    rc = quantise_w(st);
    if (rc) return rc;
    mark(K_W_QUANT);
  }
  if (!gx_aside) {
    rc = gemm_gx(st);
    if (rc) return rc;
    mark(K_GEMM_GX);
  }
  return HOT_OK;
}

// Runs the backward with an event after every kernel group and returns the K_COUNT durations (s).
static int run_backward_timed(const void* gy, const void* w, int dtype, const void* xq, const float* sx, int64_t L,
                              int64_t O, int64_t I, const hot_config* cfg, void* gx, void* gw, int out_dtype,
                              void* workspace, size_t workspace_bytes, float* secs, hipStream_t st) {
  hipEvent_t ev[K_COUNT + 1];
  int slot_of[K_COUNT];
  for (int i = 0; i <= K_COUNT; ++i) ev[i] = nullptr;
  for (int i = 0; i < K_COUNT; ++i) { slot_of[i] = -1; secs[i] = 0.f; }
  int rc = HOT_OK;
  for (int i = 0; i <= K_COUNT && !rc; ++i) rc = check_hip(hipEventCreate(&ev[i]), "hipEventCreate");
  if (!rc) rc = run_backward(gy, w, dtype, xq, sx, L, O, I, cfg, gx, gw, out_dtype, workspace, workspace_bytes, ev, slot_of, st);
  if (!rc) rc = check_hip(hipEventSynchronize(ev[K_COUNT]), "hipEventSynchronize");
  if (!rc) {
    for (int i = 0; i < K_COUNT; ++i) {
      float ms = 0.f;
      (void)hipEventElapsedTime(&ms, ev[i], ev[i + 1]);
      if (slot_of[i] >= 0) secs[slot_of[i]] = ms * 1e-3f;
    }
  }
  for (int i = 0; i <= K_COUNT; ++i)
    if (ev[i]) (void)hipEventDestroy(ev[i]);
  return rc;
}

int hot_linear_backward(const void* gy, const void* w, int dtype, const void* xq, const float* sx, int64_t L,
                        int64_t O, int64_t I, const hot_config* cfg, void* gx, void* gw, int out_dtype,
                        void* workspace, size_t workspace_bytes, float* times4, void* hip_stream) {
  if (!times4)
    return run_backward(gy, w, dtype, xq, sx, L, O, I, cfg, gx, gw, out_dtype, workspace, workspace_bytes, nullptr,
                        nullptr, (hipStream_t)hip_stream);
  float k[K_COUNT];
  const int rc = run_backward_timed(gy, w, dtype, xq, sx, L, O, I, cfg, gx, gw, out_dtype, workspace, workspace_bytes,
                                    k, (hipStream_t)hip_stream);
  if (rc) return rc;
  // the reference op returns {fwht, quant, gemm, dequant} (HLQ_backward_kernel.cu:729-733)
  times4[0] = k[K_CLEAR] + k[K_GY_STATS] + k[K_W_STATS];          // transform passes that only measure
  times4[1] = k[K_GY_HLA] + k[K_GY_HQ] + k[K_W_QUANT];            // transform + quantise passes
  times4[2] = k[K_GEMM_GX] + k[K_GEMM_GW];                        // both GEMMs
  times4[3] = 0.f;                                                // dequantisation: fused into the GEMMs' epilogues
  return HOT_OK;
}

int hot_linear_backward_bias(const void* gy, const void* w, int dtype, const void* xq, const float* sx, int64_t L,
                             int64_t O, int64_t I, const hot_config* cfg, void* gx, void* gw, void* gb, int out_dtype,
                             void* workspace, size_t workspace_bytes, void* hip_stream) {
  if (!gb) return fail(HOT_ERR_INVALID, "hot_linear_backward_bias: null pointer");
  return run_backward(gy, w, dtype, xq, sx, L, O, I, cfg, gx, gw, out_dtype, workspace, workspace_bytes, nullptr,
                      nullptr, (hipStream_t)hip_stream, gb);
}

// ---- g_x through a low-rank projection along the tokens ---------------------------------------------
// transform_scheme "low_rank" and "gilr_gwh" (utils/quant_matmul.py:229-233, 263-266, 288-290, 334-337):
// g_x = P^T ( q(P g_y) . q(W) ) s_g s_w / n, W untransformed.  The token-wise kernels store q(P g_y)
// untransposed ([L', O], K along the channels), W goes through the column-wise kernel with blocks of
// one row (quantise + transpose), the product lands in fp32 in the workspace and the expansion pass
// takes it back to L tokens.  Kept for completeness of the reference's scheme list: four kernels on
// one stream, not tuned.  The g_W side of those schemes is the g_W side of "gih_gwlr" / "hadamard".

struct LowrankLayout {
  int64_t lp, ld_g, ld_w;
  size_t off_colg, off_colw, off_sg, off_sw, off_qg, off_qw, off_t, off_exp, off_proj, colg_bytes, exp_bytes, total;
};

static LowrankLayout lowrank_layout(int64_t L, int64_t O, int64_t I, const hot_config* c) {
  LowrankLayout b;
  b.lp = (L / c->hla_n) * c->hla_r;
  b.ld_g = round_up(O, GEMM_KTILE) * c->gx_bits / 8;
  b.ld_w = round_up(O, GEMM_KTILE) * c->w_bits / 8;
  size_t o = 0;
  // blocks above 128 tokens: the two-level token-wise path and the two-pass expansion, each with an
  // fp32 intermediate of the tensor's size in the workspace
  b.colg_bytes = hla_workspace_bytes_impl(L, O, c->hla_n, c->hla_r);
  b.exp_bytes = c->hla_n > 128 ? hla_expand_big_workspace_bytes_impl(L / c->hla_n, I, c->hla_n) : 0;
  b.off_colg = o; o += align256(b.colg_bytes);
  b.off_colw = o; o += align256(colwise_workspace_bytes_impl(I));
  // a step per coefficient row (gx_scale ROW): lp steps, and the unquantised projection [L', O] in fp32
  const bool per_row = c->gx_scale == HOT_SCALE_ROW;
  b.off_sg = o;   o += per_row ? align256((size_t)b.lp * 4) : 256;
  b.off_sw = o;   o += 256;
  b.off_qg = o;   o += align256((size_t)b.lp * b.ld_g);
  b.off_qw = o;   o += align256((size_t)I * b.ld_w);
  b.off_t = o;    o += align256((size_t)b.lp * (size_t)I * 4);
  b.off_exp = o;  o += align256(b.exp_bytes);
  b.off_proj = o; o += per_row ? align256((size_t)b.lp * (size_t)O * 4) : 0;
  b.total = o;
  return b;
}

static int check_lowrank(const hot_config* cfg, int64_t L, int64_t O, int64_t I, const char* who) {
  if (int e = check_cfg(cfg, who)) return e;
  if (L <= 0 || O <= 0 || I <= 0 || O % 8 || I % 8) return fail(HOT_ERR_INVALID, "%s: L=%lld, O=%lld and I=%lld must be positive, O and I multiples of 8", who, (long long)L, (long long)O, (long long)I);
  if (L % cfg->hla_n) return fail(HOT_ERR_INVALID, "%s: L=%lld is not a multiple of hla_n=%d", who, (long long)L, cfg->hla_n);
  if (cfg->gx_bits != cfg->w_bits) return fail(HOT_ERR_UNSUPPORTED, "%s: gx_bits (%d) and w_bits (%d) must match", who, cfg->gx_bits, cfg->w_bits);
  if (cfg->gx_scale == HOT_SCALE_SAWB) return fail(HOT_ERR_UNSUPPORTED, "%s: the projected g_y takes absmax steps (one for the tensor or one per coefficient row)", who);
  if (cfg->gx_scale == HOT_SCALE_ROW && cfg->hla_n > 128) return fail(HOT_ERR_UNSUPPORTED, "%s: a step per coefficient row takes token blocks up to 128", who);
  if (cfg->w_scale == HOT_SCALE_ROW) return fail(HOT_ERR_UNSUPPORTED, "%s: W uses one step per tensor", who);
  return HOT_OK;
}

size_t hot_gx_lowrank_workspace_bytes(int64_t L, int64_t O, int64_t I, const hot_config* cfg) {
  if (check_lowrank(cfg, L, O, I, "hot_gx_lowrank_workspace_bytes")) return 0;
  return lowrank_layout(L, O, I, cfg).total;
}

int hot_gx_lowrank(const void* gy, const void* w, int dtype, int64_t L, int64_t O, int64_t I, const hot_config* cfg,
                   void* gx, int out_dtype, void* workspace, size_t workspace_bytes, void* hip_stream) {
  const char* who = "hot_gx_lowrank";
  if (int e = check_lowrank(cfg, L, O, I, who)) return e;
  if (!gy || !w || !gx) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (L * O * 4 >= (1ll << 32) || O * I * 4 >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "%s: tensors exceed the 32-bit offsets of the loader", who);
  const LowrankLayout b = lowrank_layout(L, O, I, cfg);
  if (!workspace || workspace_bytes < b.total) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, b.total, workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  hipStream_t st = (hipStream_t)hip_stream;
  uint8_t* ws = (uint8_t*)workspace;
  float* sg = (float*)(ws + b.off_sg);
  float* sw = (float*)(ws + b.off_sw);
  const int bits = cfg->gx_bits;
  // q(P g_y), untransposed [L', O]; the K padding of every row is cleared apart
  int rc;
  const bool per_row = cfg->gx_scale == HOT_SCALE_ROW;
  if (per_row) {
    // a step per coefficient row (norm_quantizer on [L', O], utils/quant_matmul.py:19-37,244-255): the
    // projection unquantised in fp32, then the row-wise quantiser without a transform (elements numbered
    // row-major for stochastic rounding)
    float* proj = (float*)(ws + b.off_proj);
    rc = hla_project_impl(gy, dtype, L, O, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, proj, O, st, true);
    if (!rc) rc = hq_rowwise_impl(proj, HOT_F32, b.lp, O, 1, bits, cfg->gx_round, cfg->seed, HOT_STREAM_GX, HOT_SCALE_ROW,
                                  ws + b.off_qg, b.ld_g, sg, nullptr, 0, st);
  } else {
    rc = colwise_quant_impl(gy, dtype, L, O, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, bits, cfg->gx_round, cfg->seed,
                            HOT_STREAM_GX, HOT_SCALE_TENSOR, ws + b.off_qg, b.ld_g, bits == 4, sg, ws + b.off_colg,
                            b.colg_bytes, st, who, nullptr, false, nullptr, nullptr, 1, 0, true);
  }
  if (rc) return rc;
  zero_pad_impl(ws + b.off_qg, b.lp, O * bits / 8, b.ld_g, st);
  // q(W), stored [I, O]: blocks of one row, nothing transformed
  rc = colwise_quant_impl(w, dtype, O, I, 1, identity_rows(), 1, cfg->w_bits, cfg->w_round, cfg->seed, HOT_STREAM_W,
                          cfg->w_scale, ws + b.off_qw, b.ld_w, cfg->w_bits == 4, sw, ws + b.off_colw,
                          colwise_workspace_bytes_impl(I), st, who);
  if (rc) return rc;
  float* t = (float*)(ws + b.off_t);
  rc = gemm_i8_impl(ws + b.off_qg, b.ld_g, ws + b.off_qw, b.ld_w, bits, b.lp, I, O, sg, per_row ? 1 : 0, sw, 1.0f, t, HOT_F32, I, nullptr, st);
  if (rc) return rc;
  if (cfg->hla_n > 128)
    return hla_expand_big_impl(t, L / cfg->hla_n, I, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, 1.0f / (float)cfg->hla_n, gx,
                               out_dtype, ws + b.off_exp, b.exp_bytes, st);
  return hla_expand_impl(t, L / cfg->hla_n, I, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, 1.0f / (float)cfg->hla_n, gx, out_dtype, st);
}

// ---- g_x with the logarithmic quantiser on g_y -----------------------------------------------------
// quantBWDGogi = "luq" (utils/quant_matmul.py:238,252-253,270,276-285,288-290,343): g_y blkdiag(H) through
// luq_quantizer_BWD, blkdiag(H) W through the weight quantiser, their integer product, the two steps,
// / n_o.  The LUQ codes are powers of two up to 2^(lev + 1) and travel as two INT8 planes (q = 16 a + b);
// W's INT4-range codes are stored as bytes and doubled into [16 w | w]; one INT8 product over twice the K.

struct LuqLayout {
  int64_t kp;
  size_t off_colw, off_slots, off_sg, off_sw, off_qg, off_qw, off_qw2, total;
};

static LuqLayout luq_layout(int64_t L, int64_t O, int64_t I) {
  LuqLayout b;
  b.kp = round_up(O, GEMM_KTILE);
  size_t o = 0;
  b.off_colw = o;  o += align256(colwise_workspace_bytes_impl(I));
  b.off_slots = o; o += STAT_SLOT_BYTES;
  b.off_sg = o;    o += 256;
  b.off_sw = o;    o += 256;
  b.off_qg = o;    o += align256((size_t)L * 2 * b.kp);
  b.off_qw = o;    o += align256((size_t)I * b.kp);
  b.off_qw2 = o;   o += align256((size_t)I * 2 * b.kp);
  b.total = o;
  return b;
}

static int check_luq(const hot_config* cfg, int64_t L, int64_t O, int64_t I, const char* who) {
  if (int e = check_cfg(cfg, who)) return e;
  if (L <= 0 || O <= 0 || I <= 0 || O % 8 || I % 8) return fail(HOT_ERR_INVALID, "%s: L=%lld, O=%lld and I=%lld must be positive, O and I multiples of 8", who, (long long)L, (long long)O, (long long)I);
  if (O % cfg->n_o) return fail(HOT_ERR_INVALID, "%s: O=%lld is not a multiple of n_o=%d", who, (long long)O, cfg->n_o);
  if (cfg->gx_bits != 4 || cfg->w_bits != 4) return fail(HOT_ERR_UNSUPPORTED, "%s: the logarithmic quantiser runs at 4 bits against 4-bit weights", who);
  if (cfg->w_scale == HOT_SCALE_ROW) return fail(HOT_ERR_UNSUPPORTED, "%s: W uses one step per tensor", who);
  return HOT_OK;
}

size_t hot_gx_luq_workspace_bytes(int64_t L, int64_t O, int64_t I, const hot_config* cfg) {
  if (check_luq(cfg, L, O, I, "hot_gx_luq_workspace_bytes")) return 0;
  return luq_layout(L, O, I).total;
}

int hot_gx_luq(const void* gy, const void* w, int dtype, int64_t L, int64_t O, int64_t I, const hot_config* cfg,
               void* gx, int out_dtype, void* workspace, size_t workspace_bytes, void* hip_stream) {
  const char* who = "hot_gx_luq";
  if (int e = check_luq(cfg, L, O, I, who)) return e;
  if (!gy || !w || !gx) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (O * I * 4 >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "%s: W exceeds the 32-bit offsets of the loader", who);
  const LuqLayout b = luq_layout(L, O, I);
  if (!workspace || workspace_bytes < b.total) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, b.total, workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  hipStream_t st = (hipStream_t)hip_stream;
  uint8_t* ws = (uint8_t*)workspace;
  float* sg = (float*)(ws + b.off_sg);
  float* sw = (float*)(ws + b.off_sw);
  // W: Hadamard along O + 4-bit quantiser, codes kept one per byte, stored [I, kp]; then [16 w | w]
  int rc = colwise_quant_impl(w, dtype, O, I, cfg->n_o, identity_rows(), cfg->n_o, cfg->w_bits, cfg->w_round, cfg->seed,
                              HOT_STREAM_W, cfg->w_scale, ws + b.off_qw, b.kp, 0, sw, ws + b.off_colw,
                              colwise_workspace_bytes_impl(I), st, who);
  if (rc) return rc;
  rc = luq_pair_impl(ws + b.off_qw, I, b.kp, ws + b.off_qw2, st);
  if (rc) return rc;
  rc = hq_luq_impl(gy, dtype, L, O, cfg->n_o, cfg->gx_bits, cfg->seed, ws + b.off_qg, b.kp, sg, ws + b.off_slots,
                   STAT_SLOT_BYTES, st);
  if (rc) return rc;
  return gemm_i8_impl(ws + b.off_qg, 2 * b.kp, ws + b.off_qw2, 2 * b.kp, 8, L, I, 2 * b.kp, sg, 0, sw,
                      1.0f / (float)cfg->n_o, gx, out_dtype, I, nullptr, st);
}

// ---- g_W with the logarithmic quantiser on the projected g_y ------------------------------------------
// quantBWDGogw = "luq", or luq_quantizer picked for a layer's g_W under quantAuto (utils/quant_matmul.py:
// 296-301, 307-314, 322-324): g_W = (luq((P g_y)^T) . q(P x)) s s_x / n.  The projection is computed
// unquantised in fp32 ([O, L'], rows padded with zeros to a multiple of 8: a zero draws code 0), the
// quantiser runs on its rows (element e = o K8 + k draws the uniforms 2 e, 2 e + 1 of stream 5), and the
// two planes of the codes (q = 16 a + b) meet the INT8 activation buffer in two products whose integer
// sums a last kernel combines: 16 acc_a + acc_b is the exact sum of q x.  Kept for completeness.

struct GwLuqLayout {
  int64_t lp, k8, kp;
  size_t off_slots, off_sg, off_proj, off_codes, off_acca, off_accb, total;
};

static GwLuqLayout gw_luq_layout(int64_t L, int64_t O, int64_t I, const hot_config* c) {
  GwLuqLayout b;
  b.lp = (L / c->hla_n) * c->hla_r;
  b.k8 = round_up(b.lp, 8);
  b.kp = round_up(b.lp, GEMM_KTILE);
  size_t o = 0;
  b.off_slots = o; o += STAT_SLOT_BYTES;
  b.off_sg = o;    o += 256;
  b.off_proj = o;  o += align256((size_t)O * b.k8 * 4);
  b.off_codes = o; o += align256((size_t)O * 2 * b.kp);
  b.off_acca = o;  o += align256((size_t)O * I * 4);
  b.off_accb = o;  o += align256((size_t)O * I * 4);
  b.total = o;
  return b;
}

static int check_gw_luq(const hot_config* cfg, int64_t L, int64_t O, int64_t I, const char* who) {
  if (int e = check_cfg(cfg, who)) return e;
  if (L <= 0 || O <= 0 || I <= 0 || I % 8) return fail(HOT_ERR_INVALID, "%s: L=%lld, O=%lld and I=%lld must be positive, I a multiple of 8", who, (long long)L, (long long)O, (long long)I);
  if (cfg->hla_n > 128) return fail(HOT_ERR_UNSUPPORTED, "%s: token blocks up to 128 (the projection pass holds a block per thread)", who);
  if (L % cfg->hla_n) return fail(HOT_ERR_INVALID, "%s: L=%lld is not a multiple of hla_n=%d", who, (long long)L, cfg->hla_n);
  if (cfg->gw_bits != 4) return fail(HOT_ERR_UNSUPPORTED, "%s: the logarithmic quantiser runs at 4 bits (gw_bits)", who);
  if ((L / cfg->hla_n) * cfg->hla_r > 16384) return fail(HOT_ERR_UNSUPPORTED, "%s: more than 16384 coefficients per channel overflow the int32 sums", who);
  return HOT_OK;
}

size_t hot_gw_luq_workspace_bytes(int64_t L, int64_t O, int64_t I, const hot_config* cfg) {
  if (check_gw_luq(cfg, L, O, I, "hot_gw_luq_workspace_bytes")) return 0;
  return gw_luq_layout(L, O, I, cfg).total;
}

int hot_gw_luq(const void* gy, int dtype, const void* xq, const float* sx, int64_t L, int64_t O, int64_t I,
               const hot_config* cfg, void* gw, int out_dtype, void* workspace, size_t workspace_bytes, void* hip_stream) {
  const char* who = "hot_gw_luq";
  if (int e = check_gw_luq(cfg, L, O, I, who)) return e;
  if (!gy || !xq || !sx || !gw) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  const GwLuqLayout b = gw_luq_layout(L, O, I, cfg);
  if (!workspace || workspace_bytes < b.total) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, b.total, workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  hipStream_t st = (hipStream_t)hip_stream;
  uint8_t* ws = (uint8_t*)workspace;
  float* sg = (float*)(ws + b.off_sg);
  float* proj = (float*)(ws + b.off_proj);
  int8_t* codes = (int8_t*)(ws + b.off_codes);
  int32_t* acc_a = (int32_t*)(ws + b.off_acca);
  int32_t* acc_b = (int32_t*)(ws + b.off_accb);
  int rc = hla_project_impl(gy, dtype, L, O, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, proj, b.k8, st);
  if (rc) return rc;
  rc = hq_luq_impl(proj, HOT_F32, O, b.k8, 1, cfg->gw_bits, cfg->seed, codes, b.kp, sg, ws + b.off_slots, STAT_SLOT_BYTES, st,
                   HOT_STREAM_LUQ_GW);
  if (rc) return rc;
  const float post = 1.0f / (float)cfg->hla_n;
  rc = gemm_i8_impl(codes, 2 * b.kp, xq, b.kp, 8, O, I, b.lp, sg, 0, sx, post, gw, out_dtype, I, acc_a, st);
  if (rc) return rc;
  rc = gemm_i8_impl(codes + b.kp, 2 * b.kp, xq, b.kp, 8, O, I, b.lp, sg, 0, sx, post, gw, out_dtype, I, acc_b, st);
  if (rc) return rc;
  return luq_combine_impl(acc_a, acc_b, O, I, sg, sx, post, gw, out_dtype, st);
}

// ---- 3-D activations: one set of steps per sample --------------------------------------------------
// The reference vmaps its quantisers over the batch dimension of [B, T, C] tensors
// (utils/quant_matmul.py:33-37,102-106,118-122), applies the token-wise transform inside each sample
// (utils/hadamard_matmul.py:143-161, 3-D branch) and returns one weight gradient per sample, which
// autograd sums (utils/quant_matmul.py:288-290,322-324).  Here the B samples are the rows [b T, (b+1) T)
// of the flattened tensors; the codes of sample b occupy K range [b kg, (b+1) kg) of the g_W operands,
// kg = hot_kpad_group(T') = T' rounded up to 128 codes, and the g_W product dequantises every sample's
// integer sums with that sample's steps before adding them up in fp32, in sample order.

struct BatchedLayout {
  int64_t ld_g, ld_w, kg, ld_gp;
  size_t off_colw, off_colg, off_hq, off_sg, off_sw, off_sgp, off_qg, off_qw, off_qgp, off_part, part_bytes, total;
};

static int64_t kpad_group(int64_t T, const hot_config* c) { return round_up((T / c->hla_n) * c->hla_r, 128); }

static BatchedLayout batched_layout(int64_t B, int64_t T, int64_t O, int64_t I, const hot_config* c) {
  BatchedLayout b;
  const int64_t L = B * T;
  b.ld_g = round_up(O, GEMM_KTILE) * c->gx_bits / 8;
  b.ld_w = round_up(O, GEMM_KTILE) * c->w_bits / 8;
  b.kg = kpad_group(T, c);
  b.ld_gp = B * b.kg;
  size_t o = 0;
  b.off_colw = o; o += align256(colwise_workspace_bytes_impl(I));
  b.off_colg = o; o += align256(colwise_group_workspace_bytes_impl(O, (int)B));
  b.off_hq = o;   o += align256((size_t)B * 128 > STAT_SLOT_BYTES ? (size_t)B * 128 : STAT_SLOT_BYTES);
  b.off_sg = o;   o += align256((size_t)L * 4);
  b.off_sw = o;   o += 256;
  b.off_sgp = o;  o += align256((size_t)B * (size_t)O * 4);
  b.off_qg = o;   o += align256((size_t)L * b.ld_g);
  b.off_qw = o;   o += align256((size_t)I * b.ld_w);
  b.off_qgp = o;  o += align256((size_t)O * b.ld_gp);
  b.part_bytes = gemm_grouped_workspace_bytes_impl(O, I, (int)B, b.kg);
  b.off_part = o; o += align256(b.part_bytes);
  b.total = o;
  return b;
}

static int check_batched(const hot_config* cfg, int64_t B, int64_t T, const char* who) {
  if (int e = check_cfg(cfg, who)) return e;
  if (B < 1 || B > 65535 || T < 1) return fail(HOT_ERR_INVALID, "%s: bad batch %lld x %lld tokens", who, (long long)B, (long long)T);
  if (cfg->hla_n > COL_MAX_N) return fail(HOT_ERR_UNSUPPORTED, "%s: token blocks up to %d inside a sample", who, COL_MAX_N);
  if (T % cfg->hla_n) return fail(HOT_ERR_INVALID, "%s: T=%lld is not a multiple of hla_n=%d", who, (long long)T, cfg->hla_n);
  return HOT_OK;
}

int64_t hot_kpad_group(int64_t T, const hot_config* cfg) {
  if (!cfg || cfg->hla_n < 1 || T < 1) return 0;
  return kpad_group(T, cfg);
}

size_t hot_abc_batched_workspace_bytes(int64_t B, int64_t T, int64_t I, const hot_config* cfg) {
  (void)T; (void)cfg;
  return colwise_group_workspace_bytes_impl(I > 0 ? I : 0, B > 0 ? (int)B : 1);
}

int hot_abc_forward_batched(const void* x, int dtype, int64_t B, int64_t T, int64_t I, const hot_config* cfg,
                            void* xq_out, float* sx_out, void* workspace, size_t workspace_bytes, void* hip_stream) {
  const char* who = "hot_abc_forward_batched";
  if (int e = check_batched(cfg, B, T, who)) return e;
  if (I <= 0) return fail(HOT_ERR_INVALID, "%s: bad shape I=%lld", who, (long long)I);
  if (cfg->act_scale == HOT_SCALE_ROW) return fail(HOT_ERR_UNSUPPORTED, "%s: the activation buffer uses one step per sample", who);
  const int64_t kg = kpad_group(T, cfg);
  return colwise_quant_impl(x, dtype, B * T, I, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, cfg->act_bits, cfg->act_round, cfg->seed,
                            HOT_STREAM_ACT, cfg->act_scale, xq_out, B * kg, 0, sx_out, workspace, workspace_bytes,
                            (hipStream_t)hip_stream, who, nullptr, false, nullptr, nullptr, (int)B, kg);
}

int hot_backward_batched_ranges(int64_t B, int64_t T, int64_t O, int64_t I, const hot_config* cfg) {
  if (check_batched(cfg, B, T, "hot_backward_batched_ranges") || O <= 0 || I <= 0) return 0;
  return gemm_grouped_splits_impl(O, I, (int)B, kpad_group(T, cfg));
}

size_t hot_backward_batched_workspace_bytes(int64_t B, int64_t T, int64_t O, int64_t I, const hot_config* cfg) {
  if (check_batched(cfg, B, T, "hot_backward_batched_workspace_bytes") || O <= 0 || I <= 0) return 0;
  return batched_layout(B, T, O, I, cfg).total;
}

int hot_linear_backward_batched(const void* gy, const void* w, int dtype, const void* xq, const float* sx, int64_t B,
                                int64_t T, int64_t O, int64_t I, const hot_config* cfg, void* gx, void* gw, int out_dtype,
                                void* workspace, size_t workspace_bytes, void* hip_stream) {
  const char* who = "hot_linear_backward_batched";
  if (int e = check_batched(cfg, B, T, who)) return e;
  if (!gy || !w || !xq || !sx || !gx || !gw) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (O <= 0 || I <= 0 || O % 8 || I % 8) return fail(HOT_ERR_INVALID, "%s: O=%lld and I=%lld must be positive multiples of 8", who, (long long)O, (long long)I);
  if (O % cfg->n_o) return fail(HOT_ERR_INVALID, "%s: O=%lld is not a multiple of n_o=%d", who, (long long)O, cfg->n_o);
  if (cfg->gx_bits != cfg->w_bits) return fail(HOT_ERR_UNSUPPORTED, "%s: gx_bits (%d) and w_bits (%d) must match", who, cfg->gx_bits, cfg->w_bits);
  if (cfg->gx_scale == HOT_SCALE_SAWB || cfg->gw_scale == HOT_SCALE_SAWB) return fail(HOT_ERR_UNSUPPORTED, "%s: SAWB applies to W and x only", who);
  if (cfg->w_scale == HOT_SCALE_ROW) return fail(HOT_ERR_UNSUPPORTED, "%s: W uses one step per tensor", who);
  const int64_t L = B * T;
  if (L * O * 4 >= (1ll << 32) || O * I * 4 >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "%s: tensors exceed the 32-bit offsets of the loader", who);
  const BatchedLayout b = batched_layout(B, T, O, I, cfg);
  if (!workspace || workspace_bytes < b.total) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, b.total, workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  hipStream_t st = (hipStream_t)hip_stream;
  uint8_t* ws = (uint8_t*)workspace;
  float* sg = (float*)(ws + b.off_sg);
  float* sw = (float*)(ws + b.off_sw);
  float* sgp = (float*)(ws + b.off_sgp);
  // W: Hadamard along O + quantise, stored [I, O]
  int rc = colwise_quant_impl(w, dtype, O, I, cfg->n_o, identity_rows(), cfg->n_o, cfg->w_bits, cfg->w_round, cfg->seed,
                              HOT_STREAM_W, cfg->w_scale, ws + b.off_qw, b.ld_w, cfg->w_bits == 4, sw, ws + b.off_colw,
                              colwise_workspace_bytes_impl(I), st, who);
  if (rc) return rc;
  // g_y: Hadamard along O, one step per sample (or per token) -> g_x operand; the GEMM reads a step per row
  rc = hq_rowwise_impl(gy, dtype, L, O, cfg->n_o, cfg->gx_bits, cfg->gx_round, cfg->seed, HOT_STREAM_GX, cfg->gx_scale,
                       ws + b.off_qg, b.ld_g, sg, ws + b.off_hq, b.off_sg - b.off_hq, st, false,
                       cfg->gx_scale == HOT_SCALE_TENSOR ? T : 0, nullptr);
  if (rc) return rc;
  rc = gemm_i8_impl(ws + b.off_qg, b.ld_g, ws + b.off_qw, b.ld_w, cfg->gx_bits, L, I, O, sg, 1, sw, 1.0f / (float)cfg->n_o, gx,
                    out_dtype, I, nullptr, st);
  if (rc) return rc;
  // g_y: HLA inside every sample, one step per sample (or per sample and channel), transposed -> g_W operand
  rc = colwise_quant_impl(gy, dtype, L, O, cfg->hla_n, cfg_rows(cfg), cfg->hla_r, cfg->gw_bits, cfg->gw_round, cfg->seed,
                          HOT_STREAM_GW, cfg->gw_scale, ws + b.off_qgp, b.ld_gp, 0, sgp, ws + b.off_colg,
                          colwise_group_workspace_bytes_impl(O, (int)B), st, who, nullptr, false, nullptr, nullptr, (int)B, b.kg);
  if (rc) return rc;
  // g_W = sum over samples of (qGp_b . xq_b^T) sGp_b sx_b / hla_n
  return gemm_i8_grouped_impl(ws + b.off_qgp, b.ld_gp, xq, b.ld_gp, O, I, (int)B, b.kg, sgp, cfg->gw_scale == HOT_SCALE_ROW, sx,
                              1.0f / (float)cfg->hla_n, gw, out_dtype, I, ws + b.off_part, b.part_bytes, st);
}

int hot_linear_backward_kernels(const void* gy, const void* w, int dtype, const void* xq, const float* sx, int64_t L,
                                int64_t O, int64_t I, const hot_config* cfg, void* gx, void* gw, int out_dtype,
                                void* workspace, size_t workspace_bytes, float* times8, void* hip_stream) {
  if (!times8) return fail(HOT_ERR_INVALID, "hot_linear_backward_kernels: null times8");
  return run_backward_timed(gy, w, dtype, xq, sx, L, O, I, cfg, gx, gw, out_dtype, workspace, workspace_bytes, times8,
                            (hipStream_t)hip_stream);
}

}  // extern "C"
