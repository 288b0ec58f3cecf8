// Expansion pass of the schemes that project g_y to low rank along the tokens for the g_x product
// (utils/quant_matmul.py:334-337, transform_scheme "low_rank" / "gilr_gwh":
// grad_input = lowering_matmul_back(h.mT, grad_input) / n): the [L', I] product goes back to [L, I]
// through P^T, block by block.  H_n is symmetric, so P^T c = H_n z with z = the r coefficients at
// their natural rows and zeros elsewhere: the same canonical butterflies as every other transform
// here (adding an exact zero changes no bit), then one exact scaling by 1 / n.
//
// A thread owns one channel; its column of the block lives in LDS ([n][threads] floats, the thread's
// own bank column, so no thread ever touches another's values and no barrier is needed; 256 threads
// up to n = 64, 128 at n = 128: 64 KiB either way).  Larger blocks: hla_expand_big_impl.  Kept for
// completeness of the reference's scheme list, not tuned: memory-bound work done at LDS speed.
#include <hip/hip_runtime.h>

#include <mutex>

#include "hot_device.h"
#include "hot_host.h"

namespace hot {

constexpr int EXP_MAX_N = 128;
constexpr int EXP_THREADS = 256;   // (at most; the launch may use fewer)

struct ExpandArgs {
  const float* t;      // [nb r, C]
  void* out;           // [nb n, C]
  int64_t nb, C;
  int32_t n, r;
  float post;
  int8_t row[EXP_MAX_N];   // natural row of the k-th coefficient
};

template <typename OutT>
__global__ void __launch_bounds__(EXP_THREADS) hla_expand_kernel(const ExpandArgs a) {
  extern __shared__ float col[];                      // [n][threads]
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t c = (int64_t)blockIdx.x * nt + tid;
  const int64_t blk = blockIdx.y;
  if (c >= a.C) return;                               // no barriers below: a thread may leave alone
  for (int i = 0; i < a.n; ++i) col[i * nt + tid] = 0.f;
  const float* src = a.t + blk * a.r * a.C + c;
  for (int k = 0; k < a.r; ++k) col[a.row[k] * nt + tid] = src[(int64_t)k * a.C];
  for (int h = 1; h < a.n; h <<= 1)
    for (int i = 0; i < a.n; ++i)
      if ((i & h) == 0) {
        const float x = col[i * nt + tid], y = col[(i + h) * nt + tid];
        col[i * nt + tid] = x + y;
        col[(i + h) * nt + tid] = x - y;
      }
  OutT* dst = reinterpret_cast<OutT*>(a.out) + blk * a.n * a.C + c;
  for (int i = 0; i < a.n; ++i) store_scalar<OutT>(dst + (int64_t)i * a.C, col[i * nt + tid] * a.post);
}

int hla_expand_impl(const float* t, int64_t nb, int64_t C, int n, const int32_t* rows, int r, float post,
                    void* out, int out_dtype, hipStream_t st) {
  const char* who = "hla_expand";
  if (!t || !out || !rows) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (nb <= 0 || C <= 0) return fail(HOT_ERR_INVALID, "%s: bad shape %lld blocks x %lld channels", who, (long long)nb, (long long)C);
  if (n < 1 || n > EXP_MAX_N || (n & (n - 1))) return fail(HOT_ERR_UNSUPPORTED, "%s: block %d (a power of two up to %d)", who, n, EXP_MAX_N);
  if (r < 1 || r > n) return fail(HOT_ERR_INVALID, "%s: r=%d outside [1, %d]", who, r, n);
  if (nb > 65535) return fail(HOT_ERR_UNSUPPORTED, "%s: more than 65535 token blocks", who);
  ExpandArgs a;
  a.t = t; a.out = out; a.nb = nb; a.C = C; a.n = n; a.r = r; a.post = post;
  bool seen[EXP_MAX_N] = {};
  for (int k = 0; k < r; ++k) {
    if (rows[k] < 0 || rows[k] >= n || seen[rows[k]]) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d out of range or listed twice", who, k, rows[k]);
    seen[rows[k]] = true;
    a.row[k] = (int8_t)rows[k];
  }
  const int nt = n > 64 ? 128 : EXP_THREADS;
  const dim3 grid((unsigned)((C + nt - 1) / nt), (unsigned)nb);
  const size_t lds = (size_t)n * nt * sizeof(float);                   // 64 KiB at n = 64 and at n = 128
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&hla_expand_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    if (attr_err == hipSuccess) attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&hla_expand_kernel<bf16_t>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    if (attr_err == hipSuccess) attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&hla_expand_kernel<f16_t>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
  });
  if (attr_err != hipSuccess) return check_hip(attr_err, "hipFuncSetAttribute(hla_expand_kernel)");
  switch (out_dtype) {
    case HOT_F32: hipLaunchKernelGGL(hla_expand_kernel<float>, grid, dim3(nt), lds, st, a); break;
    case HOT_BF16: hipLaunchKernelGGL(hla_expand_kernel<bf16_t>, grid, dim3(nt), lds, st, a); break;
    case HOT_F16: hipLaunchKernelGGL(hla_expand_kernel<f16_t>, grid, dim3(nt), lds, st, a); break;
    default: return fail(HOT_ERR_INVALID, "%s: bad out dtype %d", who, out_dtype);
  }
  return check_launch("hla_expand_kernel");
}

// ---- the projection itself, unquantised (the operand of the logarithmic quantiser on the g_W side:
// luq_quantizer(lowering_matmul_back(P, g_y).mT), utils/quant_matmul.py:296-301,307-314) ---------------
// Same ownership as the expansion: a thread holds its channel's block in its own LDS column, runs the
// canonical butterflies and writes the r kept coefficients to its channel's row of the transposed
// fp32 output.  Kept for completeness, not tuned.
struct ProjectArgs {
  const void* in;      // [nb n, C]
  float* out;          // [C, ld] (transposed) or [nb r, ld] (row-major)
  int64_t nb, C, ld;
  int32_t n, r, rowmajor;
  int8_t row[EXP_MAX_N];
};

template <typename T> __device__ __forceinline__ float load_as_f32(const void* p, int64_t i);
template <> __device__ __forceinline__ float load_as_f32<float>(const void* p, int64_t i) { return reinterpret_cast<const float*>(p)[i]; }
template <> __device__ __forceinline__ float load_as_f32<bf16_t>(const void* p, int64_t i) {
  return as_f((uint32_t)reinterpret_cast<const uint16_t*>(p)[i] << 16);
}
template <> __device__ __forceinline__ float load_as_f32<f16_t>(const void* p, int64_t i) { return (float)reinterpret_cast<const _Float16*>(p)[i]; }

template <typename T>
__global__ void __launch_bounds__(EXP_THREADS) hla_project_kernel(const ProjectArgs a) {
  extern __shared__ float col[];                      // [n][threads]
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t c = (int64_t)blockIdx.x * nt + tid;
  const int64_t blk = blockIdx.y;
  if (c >= a.C) return;                               // no barriers below
  for (int i = 0; i < a.n; ++i) col[i * nt + tid] = load_as_f32<T>(a.in, (blk * a.n + i) * a.C + c);
  for (int h = 1; h < a.n; h <<= 1)
    for (int i = 0; i < a.n; ++i)
      if ((i & h) == 0) {
        const float x = col[i * nt + tid], y = col[(i + h) * nt + tid];
        col[i * nt + tid] = x + y;
        col[(i + h) * nt + tid] = x - y;
      }
  if (a.rowmajor) {
    float* dst = a.out + blk * a.r * a.ld + c;
    for (int k = 0; k < a.r; ++k) dst[(int64_t)k * a.ld] = col[a.row[k] * nt + tid];
    return;
  }
  float* dst = a.out + c * a.ld + blk * a.r;
  for (int k = 0; k < a.r; ++k) dst[k] = col[a.row[k] * nt + tid];
  if (blk == a.nb - 1)
    for (int64_t k = a.nb * a.r; k < a.ld; ++k) a.out[c * a.ld + k] = 0.f;
}

int hla_project_impl(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows, int r, float* out,
                     int64_t ld, hipStream_t st, bool rowmajor) {
  const char* who = "hla_project";
  if (!in || !out || !rows) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (n < 1 || n > EXP_MAX_N || (n & (n - 1))) return fail(HOT_ERR_UNSUPPORTED, "%s: block %d (a power of two up to %d)", who, n, EXP_MAX_N);
  if (R <= 0 || C <= 0 || R % n) return fail(HOT_ERR_INVALID, "%s: %lld rows are not whole blocks of %d", who, (long long)R, n);
  if (r < 1 || r > n) return fail(HOT_ERR_INVALID, "%s: r=%d outside [1, %d]", who, r, n);
  const int64_t nb = R / n;
  if (nb > 65535) return fail(HOT_ERR_UNSUPPORTED, "%s: more than 65535 token blocks", who);
  if (ld < (rowmajor ? C : nb * r)) return fail(HOT_ERR_INVALID, "%s: ld=%lld too short", who, (long long)ld);
  ProjectArgs a;
  a.in = in; a.out = out; a.nb = nb; a.C = C; a.ld = ld; a.n = n; a.r = r; a.rowmajor = rowmajor ? 1 : 0;
  bool seen[EXP_MAX_N] = {};
  for (int k = 0; k < r; ++k) {
    if (rows[k] < 0 || rows[k] >= n || seen[rows[k]]) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d out of range or listed twice", who, k, rows[k]);
    seen[rows[k]] = true;
    a.row[k] = (int8_t)rows[k];
  }
  const int nt = n > 64 ? 128 : EXP_THREADS;
  const dim3 grid((unsigned)((C + nt - 1) / nt), (unsigned)nb);
  const size_t lds = (size_t)n * nt * sizeof(float);
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&hla_project_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    if (attr_err == hipSuccess) attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&hla_project_kernel<bf16_t>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    if (attr_err == hipSuccess) attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&hla_project_kernel<f16_t>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
  });
  if (attr_err != hipSuccess) return check_hip(attr_err, "hipFuncSetAttribute(hla_project_kernel)");
  switch (dtype) {
    case HOT_F32: hipLaunchKernelGGL(hla_project_kernel<float>, grid, dim3(nt), lds, st, a); break;
    case HOT_BF16: hipLaunchKernelGGL(hla_project_kernel<bf16_t>, grid, dim3(nt), lds, st, a); break;
    case HOT_F16: hipLaunchKernelGGL(hla_project_kernel<f16_t>, grid, dim3(nt), lds, st, a); break;
    default: return fail(HOT_ERR_INVALID, "%s: bad dtype %d", who, dtype);
  }
  return check_launch("hla_project_kernel");
}

template <typename OutT>
__global__ void __launch_bounds__(256) luq_combine_kernel(const int32_t* __restrict__ acc_a, const int32_t* __restrict__ acc_b,
                                                          int64_t count, const float* __restrict__ s_a,
                                                          const float* __restrict__ s_b, float post, OutT* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  const int32_t acc = 16 * acc_a[i] + acc_b[i];
  store_scalar<OutT>(out + i, (((float)acc * s_a[0]) * s_b[0]) * post);
}

int luq_combine_impl(const int32_t* acc_a, const int32_t* acc_b, int64_t M, int64_t N, const float* s_a, const float* s_b,
                     float post, void* out, int out_dtype, hipStream_t st) {
  const int64_t count = M * N;
  const dim3 grid((unsigned)((count + 255) / 256));
  switch (out_dtype) {
    case HOT_F32: hipLaunchKernelGGL(luq_combine_kernel<float>, grid, dim3(256), 0, st, acc_a, acc_b, count, s_a, s_b, post, (float*)out); break;
    case HOT_BF16: hipLaunchKernelGGL(luq_combine_kernel<bf16_t>, grid, dim3(256), 0, st, acc_a, acc_b, count, s_a, s_b, post, (bf16_t*)out); break;
    case HOT_F16: hipLaunchKernelGGL(luq_combine_kernel<f16_t>, grid, dim3(256), 0, st, acc_a, acc_b, count, s_a, s_b, post, (f16_t*)out); break;
    default: return fail(HOT_ERR_INVALID, "luq_combine: bad out dtype %d", out_dtype);
  }
  return check_launch("luq_combine_kernel");
}

}  // namespace hot
