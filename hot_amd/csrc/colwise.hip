// colwise: Hadamard transform along the ROW (strided) dimension of a row-major
// matrix, optional low-rank selection of r of the n coefficients of each
// block, quantisation, and a transposed (K-major) store for the int8 GEMM.
//
// One kernel family serves
//   * HLA of g_y and of x along the token dimension
//     (lowering_matmul_back(P, .), utils/hadamard_matmul.py:143-161 with
//      P = make_WHT :209-226; used at utils/quant_matmul.py:190 and :301), and
//   * the block-Hadamard of W along O
//     (lowering_matmul_back(H_16, W), utils/quant_matmul.py:270),
// followed by int/stoch/norm/sawb_quantizer_BWD (utils/quant_matmul.py:19-55,
// 86-122) and by the transposes the reference op feeds its GEMMs with
// (cuda_measure/HLQ_backward_kernel.cu:561,610-611).
//
// Mapping: a lane owns CPL adjacent channels (columns) and all n rows of one
// token block, so the butterflies need no cross-lane traffic and every load is
// contiguous across the wave.  The four waves of a workgroup share a channel
// group and take different token blocks; codes are staged in LDS as
// [channel][k] so that each channel's K-run leaves the CU as one contiguous
// segment.  Two passes over the input (statistics, then quantise): the scale
// of a tensor depends on all of it.
//
// HBM traffic per input element: 2 * sizeof(in) read + (r/n) * bits/8 written.
#include "hot_device.h"
#include "hot_host.h"

namespace hot {

constexpr int COL_THREADS = 256;
constexpr int COL_WAVES = COL_THREADS / 64;

struct ColArgs {
  const void* in;
  int64_t R, C;       // input rows (transform dim) and channels
  int64_t NB;         // token blocks = R / N
  int64_t Kout;       // NB * r codes per output row
  int8_t* out;
  int64_t ld_out;     // bytes
  float* stat;        // [0] absmax, [1] step s, [2] clip
  double* partial;    // SAWB: 2 doubles per workgroup
  float* colmax;      // ROW: per-channel absmax
  float* scales_out;
  uint64_t seed;
  uint32_t stream;
  int32_t r, bits, store4, rounding, mode, bpw;
  int8_t slot[HOT_MAX_HLA_N];  // output position of natural row i, -1 = dropped
};

template <int N> struct cpl_of { static constexpr int value = N >= 64 ? 2 : 4; };

template <typename T, int CPL>
__device__ __forceinline__ void load_cpl(const T* p, float* o) {
  constexpr int BYTES = CPL * (int)sizeof(T);
  if constexpr (BYTES == 4) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    if constexpr (sizeof(T) == 4) { o[0] = as_f(w); }
    else { float t[8]; unpack_vec<T>(make_uint4(w, 0, 0, 0), t); o[0] = t[0]; o[1] = t[1]; }
  } else if constexpr (BYTES == 8) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    if constexpr (sizeof(T) == 4) { o[0] = as_f(w.x); o[1] = as_f(w.y); }
    else { float t[8]; unpack_vec<T>(make_uint4(w.x, w.y, 0, 0), t); o[0] = t[0]; o[1] = t[1]; o[2] = t[2]; o[3] = t[3]; }
  } else {
    static_assert(BYTES == 16, "unsupported channels-per-lane");
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    float t[8];
    unpack_vec<T>(w, t);
#pragma unroll
    for (int i = 0; i < CPL; ++i) o[i] = t[i];
  }
}

// Loads block `blk` (N rows x CPL channels starting at channel c0) and applies
// the unnormalised FWHT along the row index, stages h = 1, 2, 4, ...
template <typename T, int N, int CPL>
__device__ __forceinline__ void load_transform(const T* in, int64_t C, int64_t blk, int64_t c0, float (&x)[N][CPL]) {
  const T* p = in + (blk * N) * C + c0;
#pragma unroll
  for (int i = 0; i < N; ++i) load_cpl<T, CPL>(p + (int64_t)i * C, x[i]);
#pragma unroll
  for (int h = 1; h < N; h <<= 1) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if ((i & h) == 0) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          const float a = x[i][c], b = x[i + h][c];
          x[i][c] = a + b;
          x[i + h][c] = a - b;
        }
      }
    }
  }
}

// ---- pass 1: statistics of the kept coefficients ------------------------------

template <typename T, int N>
__global__ void __launch_bounds__(COL_THREADS) colwise_stats_kernel(const ColArgs a) {
  constexpr int CPL = cpl_of<N>::value;
  __shared__ float s_max[COL_WAVES];
  __shared__ double s_sum[2][COL_WAVES];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t c0 = ((int64_t)blockIdx.x * 64 + lane) * CPL;
  const bool active = c0 < a.C;
  const int tb = COL_WAVES * a.bpw;
  const int64_t b0 = (int64_t)blockIdx.y * tb + (int64_t)wave * a.bpw;

  float cmax[CPL];
  double ssq = 0.0, sab = 0.0;
#pragma unroll
  for (int c = 0; c < CPL; ++c) cmax[c] = 0.f;

  for (int j = 0; j < a.bpw; ++j) {
    const int64_t blk = b0 + j;
    if (blk >= a.NB || !active) break;
    float x[N][CPL];
    load_transform<T, N, CPL>((const T*)a.in, a.C, blk, c0, x);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (a.slot[i] >= 0) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          cmax[c] = fmaxf(cmax[c], fabsf(x[i][c]));
          if (a.mode == HOT_SCALE_SAWB) { ssq += (double)x[i][c] * (double)x[i][c]; sab += (double)fabsf(x[i][c]); }
        }
      }
    }
  }

  if (a.mode == HOT_SCALE_ROW) {
    if (active) {
#pragma unroll
      for (int c = 0; c < CPL; ++c) atomic_max_nonneg(a.colmax + c0 + c, cmax[c]);
    }
    return;
  }
  if (a.mode == HOT_SCALE_TENSOR) {
    float m = 0.f;
#pragma unroll
    for (int c = 0; c < CPL; ++c) m = fmaxf(m, cmax[c]);
    m = wave_max(m);
    if (lane == 0) s_max[wave] = m;
    __syncthreads();
    if (tid == 0) {
      float mm = s_max[0];
      for (int i = 1; i < COL_WAVES; ++i) mm = fmaxf(mm, s_max[i]);
      atomic_max_nonneg(a.stat, mm);
    }
    return;
  }
  // SAWB: per-workgroup partial sums, reduced in a fixed order by the finalize kernel
  ssq = wave_sum(ssq);
  sab = wave_sum(sab);
  if (lane == 0) { s_sum[0][wave] = ssq; s_sum[1][wave] = sab; }
  __syncthreads();
  if (tid == 0) {
    double q = 0.0, b = 0.0;
    for (int i = 0; i < COL_WAVES; ++i) { q += s_sum[0][i]; b += s_sum[1][i]; }
    const int64_t wg = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
    a.partial[2 * wg] = q;
    a.partial[2 * wg + 1] = b;
  }
}

// ---- finalize: statistics -> step sizes ----------------------------------------

__global__ void __launch_bounds__(256) colwise_finalize_kernel(const ColArgs a, int64_t nwg) {
  __shared__ double s_q[256], s_b[256];
  const float qmax = (float)((1 << (a.bits - 1)) - 1);
  const int tid = threadIdx.x;
  if (a.mode == HOT_SCALE_ROW) {
    for (int64_t c = tid; c < a.C; c += 256) a.scales_out[c] = a.colmax[c] / qmax;
    return;
  }
  if (a.mode == HOT_SCALE_TENSOR) {
    if (tid == 0) {
      const float mx = a.stat[0];
      const float s = mx / qmax;
      a.stat[1] = s;
      a.stat[2] = mx;
      a.scales_out[0] = s;
    }
    return;
  }
  double q = 0.0, b = 0.0;
  for (int64_t i = tid; i < nwg; i += 256) { q += a.partial[2 * i]; b += a.partial[2 * i + 1]; }
  s_q[tid] = q; s_b[tid] = b;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) { s_q[tid] += s_q[tid + s]; s_b[tid] += s_b[tid + s]; }
    __syncthreads();
  }
  if (tid == 0) {
    const double cnt = (double)a.Kout * (double)a.C;
    const float clip = (float)(12.1 * sqrt(s_q[0] / cnt) - 12.2 * (s_b[0] / cnt));
    const float s = clip / qmax;
    a.stat[1] = s;
    a.stat[2] = clip;
    a.scales_out[0] = s;
  }
}

// ---- pass 2: transform again, quantise, transpose through LDS, store --------

template <typename T, int N, int ROUND, bool SAWB>
__global__ void __launch_bounds__(COL_THREADS) colwise_quant_kernel(const ColArgs a) {
  constexpr int CPL = cpl_of<N>::value;
  constexpr int CG = 64 * CPL;  // channels per workgroup
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tb = COL_WAVES * a.bpw;
  const int sb = tb * a.r;           // code bytes per channel in LDS
  const int pitch = sb + 4;          // odd dword pitch for even sb/4 .. keeps byte writes spread over banks
  const int64_t cg0 = (int64_t)blockIdx.x * CG;
  const int64_t c0 = cg0 + (int64_t)lane * CPL;
  const bool active = c0 < a.C;
  const int64_t b0 = (int64_t)blockIdx.y * tb + (int64_t)wave * a.bpw;
  const int qmax = (1 << (a.bits - 1)) - 1;

  // zero the staging area (partial token-block groups leave gaps that must read as 0)
  {
    uint32_t* l32 = reinterpret_cast<uint32_t*>(lds);
    const int n32 = CG * pitch / 4;
    for (int i = tid; i < n32; i += COL_THREADS) l32[i] = 0u;
  }
  __syncthreads();

  float d[CPL], clip = 0.f;
  if (a.mode == HOT_SCALE_ROW) {
#pragma unroll
    for (int c = 0; c < CPL; ++c) d[c] = active ? (a.colmax[c0 + c] / (float)qmax + 1e-11f) : 1.f;
  } else {
    const float s = a.stat[1];
    clip = a.stat[2];
#pragma unroll
    for (int c = 0; c < CPL; ++c) d[c] = s + 1e-11f;
  }

  for (int j = 0; j < a.bpw; ++j) {
    const int64_t blk = b0 + j;
    if (blk >= a.NB || !active) break;
    float x[N][CPL];
    load_transform<T, N, CPL>((const T*)a.in, a.C, blk, c0, x);
    const int kl0 = (wave * a.bpw + j) * a.r;  // position of this block inside the staged run
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int sl = a.slot[i];
      if (sl >= 0) {
        float u[4];
        if constexpr (ROUND == HOT_ROUND_STOCH) {
          // element index of coefficient (k, c) is k * C + c; c0 is a multiple of CPL, so the
          // lane's channels share one (CPL = 4) or half of one (CPL = 2) counter value
          const uint64_t e = (uint64_t)(blk * a.r + sl) * (uint64_t)a.C + (uint64_t)c0;
          sr_uniform4(e >> 2, a.seed, a.stream, u);
        }
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          float v = x[i][c];
          if constexpr (SAWB) v = fminf(fmaxf(v, -clip), clip);
          const float y = v / d[c];
          int q;
          if constexpr (ROUND == HOT_ROUND_NEAREST) {
            q = q_nearest(y);
          } else {
            q = q_stoch(y, CPL == 4 ? u[c] : ((c0 & 2) ? u[2 + c] : u[c]));
          }
          q = clampi(q, -qmax, qmax);
          lds[(lane * CPL + c) * pitch + kl0 + sl] = (uint8_t)(q & 0xFF);
        }
      }
    }
  }
  __syncthreads();

  // flush: each channel's staged run is one contiguous global segment
  const bool last = (int64_t)(blockIdx.y + 1) * tb >= a.NB;
  const int64_t seg0 = (int64_t)blockIdx.y * (a.store4 ? sb / 2 : sb);  // byte offset in the output row
  const int64_t seg_end = last ? a.ld_out : seg0 + (a.store4 ? sb / 2 : sb);
  const int ndw = (int)((seg_end - seg0) / 4);  // output dwords per channel
  const int sdw = (a.store4 ? sb / 2 : sb) / 4; // of which staged
  const int64_t nch = (a.C - cg0) < CG ? (a.C - cg0) : CG;
  for (int64_t p = tid; p < nch * ndw; p += COL_THREADS) {
    const int ch = (int)(p / ndw), jd = (int)(p % ndw);
    uint32_t w = 0u;
    if (jd < sdw) {
      const uint32_t* row = reinterpret_cast<const uint32_t*>(lds + ch * pitch);
      if (a.store4) {
        const uint32_t lo = row[2 * jd], hi = row[2 * jd + 1];
        // bytes b0..b7 -> nibbles: byte j of the result = (b[2j+1] << 4) | (b[2j] & 15)
        const uint32_t l = (lo & 0x0F) | ((lo >> 4) & 0xF0) | ((lo >> 8) & 0x0F00) | ((lo >> 12) & 0xF000);
        const uint32_t h = (hi & 0x0F) | ((hi >> 4) & 0xF0) | ((hi >> 8) & 0x0F00) | ((hi >> 12) & 0xF000);
        w = (l & 0xFFFF) | (h << 16);
      } else {
        w = row[jd];
      }
    }
    *reinterpret_cast<uint32_t*>(a.out + (cg0 + ch) * a.ld_out + seg0 + (int64_t)jd * 4) = w;
  }
}

__global__ void colwise_clear_kernel(float* stat, float* colmax, int64_t C) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < 4) stat[i] = 0.f;
  if (colmax && i < C) colmax[i] = 0.f;
}

// ---- host ---------------------------------------------------------------------

static constexpr size_t COL_STAT_BYTES = 256;

size_t colwise_workspace_bytes_impl(int64_t C) {
  // stat | per-channel max | per-workgroup partial sums (worst-case count bounded on launch)
  return COL_STAT_BYTES + (size_t)round_up(C * 4, 256) + (size_t)(2 * sizeof(double)) * 65536;
}

template <typename T, int N>
static int launch_colwise(ColArgs& a, hipStream_t st) {
  constexpr int CPL = cpl_of<N>::value;
  constexpr int CG = 64 * CPL;
  // token blocks per wave: staged run of about 256 bytes per channel, LDS <= 48 KiB
  int bpw = 8;
  while (bpw > 1 && (COL_WAVES * bpw * a.r > 288 || (int64_t)CG * (COL_WAVES * bpw * a.r + 4) > 48 * 1024)) bpw >>= 1;
  if ((int64_t)CG * (COL_WAVES * bpw * a.r + 4) > 64 * 1024) return fail(HOT_ERR_UNSUPPORTED, "colwise: staging does not fit LDS");
  a.bpw = bpw;
  const int tb = COL_WAVES * bpw;
  const int64_t gx = (a.C + CG - 1) / CG, gy = (a.NB + tb - 1) / tb;
  if (gy > 65535 || gx * gy > 65536) return fail(HOT_ERR_UNSUPPORTED, "colwise: grid %lld x %lld too large", (long long)gx, (long long)gy);
  const dim3 grid((unsigned)gx, (unsigned)gy), block(COL_THREADS);
  const size_t lds = (size_t)CG * (tb * a.r + 4);
  const int64_t nclr = a.C > 4 ? a.C : 4;
  hipLaunchKernelGGL(colwise_clear_kernel, dim3((unsigned)((nclr + 255) / 256)), dim3(256), 0, st, a.stat,
                     a.mode == HOT_SCALE_ROW ? a.colmax : (float*)nullptr, a.C);
  hipLaunchKernelGGL((colwise_stats_kernel<T, N>), grid, block, 0, st, a);
  hipLaunchKernelGGL(colwise_finalize_kernel, dim3(1), dim3(256), 0, st, a, gx * gy);
  if (a.rounding == HOT_ROUND_STOCH) {
    if (a.mode == HOT_SCALE_SAWB) hipLaunchKernelGGL((colwise_quant_kernel<T, N, 1, true>), grid, block, lds, st, a);
    else hipLaunchKernelGGL((colwise_quant_kernel<T, N, 1, false>), grid, block, lds, st, a);
  } else {
    if (a.mode == HOT_SCALE_SAWB) hipLaunchKernelGGL((colwise_quant_kernel<T, N, 0, true>), grid, block, lds, st, a);
    else hipLaunchKernelGGL((colwise_quant_kernel<T, N, 0, false>), grid, block, lds, st, a);
  }
  return check_launch("colwise_quant_kernel");
}

template <typename T>
static int dispatch_colwise_n(int n, ColArgs& a, hipStream_t st) {
  switch (n) {
    case 1: return launch_colwise<T, 1>(a, st);
    case 2: return launch_colwise<T, 2>(a, st);
    case 4: return launch_colwise<T, 4>(a, st);
    case 8: return launch_colwise<T, 8>(a, st);
    case 16: return launch_colwise<T, 16>(a, st);
    case 32: return launch_colwise<T, 32>(a, st);
    case 64: return launch_colwise<T, 64>(a, st);
    default: return fail(HOT_ERR_UNSUPPORTED, "colwise: block size %d (power of two up to %d)", n, HOT_MAX_HLA_N);
  }
}

int colwise_quant_impl(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows, int r,
                       int bits, int rounding, uint64_t seed, uint32_t rng_stream, int scale_mode,
                       void* codes_out, int64_t ld_out, int store4, float* scales_out, void* workspace,
                       size_t workspace_bytes, hipStream_t st, const char* who) {
  if (!in || !codes_out || !scales_out || !rows) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (R <= 0 || C <= 0) return fail(HOT_ERR_INVALID, "%s: bad shape R=%lld C=%lld", who, (long long)R, (long long)C);
  if (n < 1 || n > HOT_MAX_HLA_N || (n & (n - 1))) return fail(HOT_ERR_UNSUPPORTED, "%s: block size %d (power of two up to %d)", who, n, HOT_MAX_HLA_N);
  if (R % n) return fail(HOT_ERR_INVALID, "%s: R=%lld is not a multiple of the block %d", who, (long long)R, n);
  if (r < 1 || r > n) return fail(HOT_ERR_INVALID, "%s: r=%d outside [1, %d]", who, r, n);
  if (bits != 4 && bits != 8) return fail(HOT_ERR_UNSUPPORTED, "%s: bits=%d (4 or 8)", who, bits);
  if (rounding != HOT_ROUND_NEAREST && rounding != HOT_ROUND_STOCH) return fail(HOT_ERR_INVALID, "%s: bad rounding %d", who, rounding);
  if (scale_mode < HOT_SCALE_TENSOR || scale_mode > HOT_SCALE_SAWB) return fail(HOT_ERR_INVALID, "%s: bad scale mode %d", who, scale_mode);
  if (C % 4) return fail(HOT_ERR_UNSUPPORTED, "%s: channel count %lld must be a multiple of 4", who, (long long)C);
  if (((uintptr_t)in & 15) || ((uintptr_t)codes_out & 15)) return fail(HOT_ERR_INVALID, "%s: pointers must be 16-byte aligned", who);

  ColArgs a;
  a.in = in; a.R = R; a.C = C; a.NB = R / n; a.Kout = a.NB * r;
  a.out = (int8_t*)codes_out; a.ld_out = ld_out;
  a.seed = seed; a.stream = rng_stream;
  a.r = r; a.bits = bits; a.rounding = rounding; a.mode = scale_mode; a.bpw = 1;
  for (int i = 0; i < HOT_MAX_HLA_N; ++i) a.slot[i] = -1;
  for (int k = 0; k < r; ++k) {
    if (rows[k] < 0 || rows[k] >= n) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d outside [0, %d)", who, k, rows[k], n);
    if (a.slot[rows[k]] != -1) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d listed twice", who, k, rows[k]);
    a.slot[rows[k]] = (int8_t)k;
  }
  const int64_t row_bytes = store4 ? a.Kout / 2 : a.Kout;
  if (store4 && (r & 1)) return fail(HOT_ERR_UNSUPPORTED, "%s: packed INT4 output needs an even r", who);
  if (ld_out < row_bytes || (ld_out & 15)) return fail(HOT_ERR_INVALID, "%s: ld_out=%lld must be a multiple of 16 and >= %lld", who, (long long)ld_out, (long long)row_bytes);
  if (!workspace || workspace_bytes < colwise_workspace_bytes_impl(C)) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed", who, colwise_workspace_bytes_impl(C));
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  a.store4 = store4;
  uint8_t* ws = (uint8_t*)workspace;
  a.stat = (float*)ws;
  a.colmax = (float*)(ws + COL_STAT_BYTES);
  a.partial = (double*)(ws + COL_STAT_BYTES + round_up(C * 4, 256));
  a.scales_out = scales_out;
  switch (dtype) {
    case HOT_F32: return dispatch_colwise_n<float>(n, a, st);
    case HOT_BF16: return dispatch_colwise_n<bf16_t>(n, a, st);
    case HOT_F16: return dispatch_colwise_n<f16_t>(n, a, st);
    default: return fail(HOT_ERR_INVALID, "%s: bad dtype %d", who, dtype);
  }
}

}  // namespace hot
