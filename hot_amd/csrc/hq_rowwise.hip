// hq_rowwise: block-Hadamard along the contiguous dimension fused with the
// absmax step and INT4/INT8 quantisation.
//
// Replaces fwht_kernel / find_scale_kernel / quant_int4(_per_token)_kernel /
// quant_int8_kernel of the reference CUDA op
// (cuda_measure/HLQ_backward_kernel.cu:39-178,282-307) with the numerics of
// lowering_matmul_front + int/stoch/norm_quantizer_BWD
// (utils/hadamard_matmul.py:121-141, utils/quant_matmul.py:19-31,86-116).
//
// Data movement: every lane owns EPL = 8 consecutive elements (one 16-byte
// load for 16-bit inputs, two for fp32), so a wave reads contiguous memory.
// Butterfly stages h < 8 run in registers, stages h >= 8 exchange with lane
// (lane ^ h/8) through DPP quad permutes or the LDS crossbar.  The stage order
// h = 1, 2, 4, ... and the (x+y, x-y) convention are those of the reference
// fwht_kernel (:63-78), which fixes the fp32 summation order.
//
// HBM traffic per element: sizeof(in) read once + bits/8 written; per-row
// scales add 4 bytes per row.  Per-tensor scales need the global absmax first,
// which costs a second read of the input.
#include "hot_device.h"
#include "hot_host.h"

namespace hot {

static_assert(STAT_SLOT_BYTES == HOT_HQ_WORKSPACE_BYTES, "the public workspace size of hot_hq_rowwise is the slot array");

constexpr int EPL = 8;  // elements per lane-chunk

template <typename T>
__device__ __forceinline__ void load_chunk(const T* p, float* x) {
  constexpr int EPV = vec_traits<T>::EPV;
  const uint4* v = reinterpret_cast<const uint4*>(p);
#pragma unroll
  for (int i = 0; i < EPL / EPV; ++i) {
    const uint4 raw = v[i];
    unpack_vec<T>(raw, x + i * EPV);
  }
}

// FWHT of the N-element blocks formed by N/EPL adjacent lanes.  N = 8 stands for every block that
// fits one lane's chunk: its actual size `nrt` (1, 2, 4 or 8) arrives at run time.
template <int N>
__device__ __forceinline__ void fwht_lanes(float* x, int lane, int nrt) {
#pragma unroll
  for (int h = 1; h < EPL; h <<= 1) {
    if (N > EPL || h < nrt) {   // no early exit: the stage loop must unroll for x to stay in registers
#pragma unroll
      for (int j = 0; j < EPL; ++j) {
        if ((j & h) == 0) {
          const float a = x[j], b = x[j + h];
          x[j] = a + b;
          x[j + h] = a - b;
        }
      }
    }
  }
  // lower lane: own + partner ; upper lane: partner - own  ==  partner + (-own)
  if constexpr (N >= 16) {
    const uint32_t sg = (lane & 1) ? 0x80000000u : 0u;
#pragma unroll
    for (int j = 0; j < EPL; ++j) x[j] = as_f(as_u(x[j]) ^ sg) + lane_xor<1>(x[j]);
  }
  if constexpr (N >= 32) {
    const uint32_t sg = (lane & 2) ? 0x80000000u : 0u;
#pragma unroll
    for (int j = 0; j < EPL; ++j) x[j] = as_f(as_u(x[j]) ^ sg) + lane_xor<2>(x[j]);
  }
  if constexpr (N >= 64) {
    const uint32_t sg = (lane & 4) ? 0x80000000u : 0u;
#pragma unroll
    for (int j = 0; j < EPL; ++j) x[j] = as_f(as_u(x[j]) ^ sg) + lane_xor<4>(x[j]);
  }
}

template <int BITS, int ROUND>
__device__ __forceinline__ void quant_store_chunk(const float* x, float d, float rcp, uint64_t e0, uint64_t seed,
                                                  uint32_t stream, int8_t* out_row_chunk) {
  constexpr int QMAX = (1 << (BITS - 1)) - 1;
  int q[EPL];
  if constexpr (ROUND == 0) {
    // |x / d| <= qmax (1 + 2^-22) because d comes from the absmax: no clamp needed
#pragma unroll
    for (int j = 0; j < EPL; ++j) q[j] = (int)rint_div_fast(x[j], d, rcp);
  } else {
    uint32_t r[EPL];
    sr_bits8(e0 >> 3, seed, stream, r);          // e0 is a multiple of EPL = 8
    const float rcpk = rcp * 65536.0f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) q[j] = q_stoch_fix(x[j], rcpk, r[j], QMAX);
  }
  if constexpr (BITS == 4) {
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < EPL; ++j) w |= (uint32_t)(q[j] & 0xF) << (4 * j);
    *reinterpret_cast<uint32_t*>(out_row_chunk) = w;
  } else {
    uint32_t w0 = 0, w1 = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      w0 |= (uint32_t)(q[j] & 0xFF) << (8 * j);
      w1 |= (uint32_t)(q[j + 4] & 0xFF) << (8 * j);
    }
    *reinterpret_cast<uint2*>(out_row_chunk) = make_uint2(w0, w1);
  }
}

// ---- per-row scales: one workgroup per row, row resident in registers ------

template <typename T, int N, int BITS, int ROUND, int C>
__global__ void hq_row_kernel(const T* __restrict__ in, int64_t K, int8_t* __restrict__ codes, int64_t ld,
                              float* __restrict__ scales, uint64_t seed, uint32_t stream, int nrt) {
  __shared__ float s_red[16];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int team = blockDim.x;
  const int64_t row = blockIdx.x;
  const int nch = (int)(K / EPL);
  const T* rp = in + row * K;

  float x[C][EPL];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int ch = tid + c * team;
    if (ch < nch) {
      load_chunk<T>(rp + (int64_t)ch * EPL, x[c]);
    } else {
#pragma unroll
      for (int j = 0; j < EPL; ++j) x[c][j] = 0.f;
    }
  }
  float mx = 0.f;
#pragma unroll
  for (int c = 0; c < C; ++c) {
    fwht_lanes<N>(x[c], lane, nrt);
#pragma unroll
    for (int j = 0; j < EPL; ++j) mx = fmaxf(mx, fabsf(x[c][j]));
  }
  mx = wave_max(mx);
  if (team > 64) {
    if (lane == 0) s_red[tid >> 6] = mx;
    __syncthreads();
    const int nw = team >> 6;
    float m = s_red[0];
    for (int i = 1; i < nw; ++i) m = fmaxf(m, s_red[i]);
    mx = m;
  }
  constexpr float QMAXF = (float)((1 << (BITS - 1)) - 1);
  const float s = mx / QMAXF;
  const float d = s + 1e-11f;
  const float rcp = 1.0f / d;
  if (tid == 0) scales[row] = s;

  int8_t* orow = codes + row * ld;
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int ch = tid + c * team;
    if (ch < nch) {
      quant_store_chunk<BITS, ROUND>(x[c], d, rcp, (uint64_t)row * (uint64_t)K + (uint64_t)ch * EPL, seed,
                                     stream, orow + (int64_t)ch * (EPL * BITS / 8));
    }
  }
}

// ---- per-tensor scale, pass 1: absmax of the transformed tensor -----------

template <typename T, int N>
__global__ void hq_absmax_kernel(const T* __restrict__ in, int64_t nchunks, float* __restrict__ absmax, int nrt) {
  __shared__ float s_red[16];
  const int lane = threadIdx.x & 63;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  float mx = 0.f;
  for (int64_t ch = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; ch < nchunks; ch += stride) {
    float x[EPL];
    load_chunk<T>(in + ch * EPL, x);
    fwht_lanes<N>(x, lane, nrt);
#pragma unroll
    for (int j = 0; j < EPL; ++j) mx = fmaxf(mx, fabsf(x[j]));
  }
  mx = wave_max(mx);
  if (lane == 0) s_red[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = s_red[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) m = fmaxf(m, s_red[i]);
    stat_slot_update(absmax, blockIdx.x, m);
  }
}

// ---- per-tensor scale, pass 2: transform again and quantise ----------------

template <typename T, int N, int BITS, int ROUND>
__global__ void hq_tensor_kernel(const T* __restrict__ in, int64_t nchunks, int64_t nch_row, int64_t ld,
                                 const float* __restrict__ absmax, int8_t* __restrict__ codes,
                                 float* __restrict__ scale_out, uint64_t seed, uint32_t stream, int nrt) {
  const int lane = threadIdx.x & 63;
  constexpr float QMAXF = (float)((1 << (BITS - 1)) - 1);
  const float s = stat_slots_max(absmax, lane) / QMAXF;   // absmax: STAT_SLOTS partial maxima
  const float d = s + 1e-11f;
  const float rcp = 1.0f / d;
  if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = s;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t ch = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; ch < nchunks; ch += stride) {
    float x[EPL];
    load_chunk<T>(in + ch * EPL, x);
    fwht_lanes<N>(x, lane, nrt);
    int64_t off = ch * (EPL * BITS / 8);
    if (ld != nch_row * (EPL * BITS / 8)) {  // padded rows
      const int64_t row = ch / nch_row;
      off = row * ld + (ch - row * nch_row) * (EPL * BITS / 8);
    }
    quant_store_chunk<BITS, ROUND>(x, d, rcp, (uint64_t)ch * EPL, seed, stream, codes + off);
  }
}

// ---- one scale per group of rows (3-D activations: a group is a sample) -------------------------
// The absmax of group g is collected at gmax[g * GROUP_STAT_STRIDE]: a 128-byte line per group, since
// every workgroup of a group updates it and updates of one line queue up at the memory side.
constexpr int GROUP_STAT_STRIDE = 32;
// grid (blocks per group, groups); a block walks its group's chunks with a stride of the group's blocks

template <typename T, int N>
__global__ void hq_group_absmax_kernel(const T* __restrict__ in, int64_t chunks_per_group, float* __restrict__ gmax, int nrt) {
  __shared__ float s_red[16];
  const int lane = threadIdx.x & 63;
  const int64_t g = blockIdx.y;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  float mx = 0.f;
  for (int64_t ch = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; ch < chunks_per_group; ch += stride) {
    float x[EPL];
    load_chunk<T>(in + (g * chunks_per_group + ch) * EPL, x);
    fwht_lanes<N>(x, lane, nrt);
#pragma unroll
    for (int j = 0; j < EPL; ++j) mx = fmaxf(mx, fabsf(x[j]));
  }
  mx = wave_max(mx);
  if (lane == 0) s_red[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = s_red[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) m = fmaxf(m, s_red[i]);
    atomic_max_nonneg(gmax + g * GROUP_STAT_STRIDE, m);
  }
}

// scales_out [M]: the step of every row (= of its group), the form the GEMM epilogue reads;
// group_steps [groups] (may be null): the steps themselves
template <typename T, int N, int BITS, int ROUND>
__global__ void hq_group_quant_kernel(const T* __restrict__ in, int64_t chunks_per_group, int64_t nch_row, int64_t ld,
                                      const float* __restrict__ gmax, int8_t* __restrict__ codes,
                                      float* __restrict__ scales_out, float* __restrict__ group_steps, uint64_t seed,
                                      uint32_t stream, int nrt) {
  const int lane = threadIdx.x & 63;
  const int64_t g = blockIdx.y;
  constexpr float QMAXF = (float)((1 << (BITS - 1)) - 1);
  const float s = gmax[g * GROUP_STAT_STRIDE] / QMAXF;
  const float d = s + 1e-11f;
  const float rcp = 1.0f / d;
  if (group_steps && blockIdx.x == 0 && threadIdx.x == 0) group_steps[g] = s;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t c0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c0 < chunks_per_group; c0 += stride) {
    const int64_t ch = g * chunks_per_group + c0;
    float x[EPL];
    load_chunk<T>(in + ch * EPL, x);
    fwht_lanes<N>(x, lane, nrt);
    const int64_t row = ch / nch_row, col = ch - row * nch_row;
    if (col == 0) scales_out[row] = s;
    quant_store_chunk<BITS, ROUND>(x, d, rcp, (uint64_t)ch * EPL, seed, stream, codes + row * ld + col * (EPL * BITS / 8));
  }
}

// ---- logarithmic unbiased quantiser (luq_quantizer_BWD, utils/quant_matmul.py:58-77) ---------------
// s = max(t) / 2^lev (the maximum, not the largest magnitude), lev = 2^(bits-1) - 1.  A magnitude below
// s becomes s with probability |t| / s, else 0; a magnitude m s with 2^k <= m < 2^(k+1) becomes 2^k s
// or 2^(k+1) s, the larger with probability m / 2^k - 1 (noise = 2^k (u2 - 1/2); 2^floor(log2((m + noise)
// 4 / 3)), never below 2^k).  The codes are 0 or +-2^j in units of s, j up to lev + 1 (more for negative
// elements beyond the maximum): not an INT4 / INT8 grid.  For the integer GEMM every code q is split as
// q = 16 a + b and stored in two planes of a row, a in bytes [0, Kp) and b in bytes [Kp, 2 Kp); the other
// operand carries 16 w in its first plane and w in its second, so one INT8 product over 2 Kp codes
// is the exact sum of q w.  Element e draws the uniforms 2 e and 2 e + 1 of the stream.
constexpr uint32_t LUQ_STREAM = 4;      // the g_y operand of the g_x product
constexpr uint32_t LUQ_GW_STREAM = 5;   // the projected g_y operand of the g_W product

__device__ __forceinline__ int luq_code(float x, float s, float u1, float u2) {
#pragma clang fp contract(off)
  const float ax = fabsf(x);
  if (!(s > 0.f) || x == 0.f || ax < s * u1) return 0;
  const float m = (ax < s ? s : ax) / s;                       // >= 1
  const int k = (int)((as_u(m) >> 23) & 0xFFu) - 127;          // floor(log2 m)
  const float noise = as_f((uint32_t)(k + 127) << 23) * (u2 - 0.5f);
  const float v = ((m + noise) * 4.0f) / 3.0f;
  int j = (int)((as_u(v) >> 23) & 0xFFu) - 127;
  j = j < k ? k : j;
  j = j > 10 ? 10 : j;                                         // 16 a + b with a <= 127 holds up to 2^10
  const int q = 1 << j;
  return x < 0.f ? -q : q;
}

template <typename T, int N>
__global__ void hq_posmax_kernel(const T* __restrict__ in, int64_t nchunks, float* __restrict__ slots, int nrt) {
  __shared__ float s_red[16];
  const int lane = threadIdx.x & 63;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  float mx = 0.f;
  for (int64_t ch = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; ch < nchunks; ch += stride) {
    float x[EPL];
    load_chunk<T>(in + ch * EPL, x);
    fwht_lanes<N>(x, lane, nrt);
#pragma unroll
    for (int j = 0; j < EPL; ++j) mx = fmaxf(mx, x[j]);
  }
  mx = wave_max(mx);
  if (lane == 0) s_red[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = s_red[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) m = fmaxf(m, s_red[i]);
    stat_slot_update(slots, blockIdx.x, m);
  }
}

template <typename T, int N>
__global__ void hq_luq_kernel(const T* __restrict__ in, int64_t nchunks, int64_t nch_row, int64_t ld, int64_t kp,
                              const float* __restrict__ slots, float inv_levels, int8_t* __restrict__ codes,
                              float* __restrict__ scale_out, uint64_t seed, uint32_t rng_stream, int nrt) {
  const int lane = threadIdx.x & 63;
  const float s = stat_slots_max(slots, lane) * inv_levels;       // a power of two: exact
  if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = s;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t ch = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; ch < nchunks; ch += stride) {
    float x[EPL];
    load_chunk<T>(in + ch * EPL, x);
    fwht_lanes<N>(x, lane, nrt);
    float u[2 * EPL];
    sr_uniform8((uint64_t)ch * 2, seed, rng_stream, u);          // uniforms 16 ch .. 16 ch + 15
    sr_uniform8((uint64_t)ch * 2 + 1, seed, rng_stream, u + EPL);
    uint32_t hi0 = 0, hi1 = 0, lo0 = 0, lo1 = 0;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      const int q = luq_code(x[j], s, u[2 * j], u[2 * j + 1]);
      const int mag = q < 0 ? -q : q;
      const int a = q < 0 ? -(mag >> 4) : (mag >> 4), b = q < 0 ? -(mag & 15) : (mag & 15);
      if (j < 4) { hi0 |= (uint32_t)(a & 0xFF) << (8 * j); lo0 |= (uint32_t)(b & 0xFF) << (8 * j); }
      else { hi1 |= (uint32_t)(a & 0xFF) << (8 * (j - 4)); lo1 |= (uint32_t)(b & 0xFF) << (8 * (j - 4)); }
    }
    const int64_t row = ch / nch_row, col = ch - row * nch_row;
    int8_t* o = codes + row * ld + col * EPL;
    *reinterpret_cast<uint2*>(o) = make_uint2(hi0, hi1);
    *reinterpret_cast<uint2*>(o + kp) = make_uint2(lo0, lo1);
  }
}

// second operand of a product with two-plane LUQ codes: [16 w | w] from INT8-stored codes w in [-8, 7]
__global__ void luq_pair_kernel(const int8_t* __restrict__ qw, int64_t rows, int64_t kp, int8_t* __restrict__ out) {
  const int64_t nq = kp / 16;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * nq) return;
  const int64_t row = i / nq, c = (i - row * nq) * 16;
  const uint4 v = *reinterpret_cast<const uint4*>(qw + row * kp + c);
  uint4 h;
  h.x = (v.x << 4) & 0xF0F0F0F0u; h.y = (v.y << 4) & 0xF0F0F0F0u;
  h.z = (v.z << 4) & 0xF0F0F0F0u; h.w = (v.w << 4) & 0xF0F0F0F0u;
  *reinterpret_cast<uint4*>(out + row * 2 * kp + c) = h;
  *reinterpret_cast<uint4*>(out + row * 2 * kp + kp + c) = v;
}

// zero the bytes [row_bytes, ld) of every row (K padding for the GEMM)
__global__ void zero_pad_kernel(int8_t* codes, int64_t M, int64_t row_bytes, int64_t ld) {
  const int64_t padw = (ld - row_bytes) / 4;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= M * padw) return;
  const int64_t row = i / padw, j = i - row * padw;
  *reinterpret_cast<uint32_t*>(codes + row * ld + row_bytes + j * 4) = 0u;
}

__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

void zero_pad_impl(void* codes, int64_t rows, int64_t row_bytes, int64_t ld, hipStream_t st) {
  if (ld <= row_bytes || rows <= 0) return;
  const int64_t n = rows * ((ld - row_bytes) / 4);
  hipLaunchKernelGGL(zero_pad_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (int8_t*)codes, rows, row_bytes, ld);
}

// ---- host dispatch -----------------------------------------------------------

template <typename T, int N, int BITS, int ROUND>
static int launch_row(const void* in, int64_t M, int64_t K, void* codes, int64_t ld, float* scales, uint64_t seed,
                      uint32_t stream_id, hipStream_t st, int nrt) {
  const int64_t nch = K / EPL;
  int team = 64;
  while (team < 1024 && nch > 4 * (int64_t)team) team <<= 1;
  const int64_t c = (nch + team - 1) / team;
  if (c > 8) return fail(HOT_ERR_UNSUPPORTED, "hot_hq_rowwise: K=%lld too large for per-row scales (max 65536)", (long long)K);
  const dim3 grid((unsigned)M), block(team);
#define HOT_ROW_CASE(CC)                                                                              \
  hipLaunchKernelGGL((hq_row_kernel<T, N, BITS, ROUND, CC>), grid, block, 0, st, (const T*)in, K, \
                     (int8_t*)codes, ld, scales, seed, stream_id, nrt)
  switch (c) {
    case 1: HOT_ROW_CASE(1); break;
    case 2: HOT_ROW_CASE(2); break;
    case 3: HOT_ROW_CASE(3); break;
    case 4: HOT_ROW_CASE(4); break;
    case 5: case 6: HOT_ROW_CASE(6); break;
    default: HOT_ROW_CASE(8); break;
  }
#undef HOT_ROW_CASE
  return check_launch("hq_row_kernel");
}

template <typename T, int N, int BITS, int ROUND>
static int launch_tensor(const void* in, int64_t M, int64_t K, void* codes, int64_t ld, float* scales, float* absmax,
                         uint64_t seed, uint32_t stream_id, hipStream_t st, bool absmax_ready, int nrt) {
  const int64_t nch = M * K / EPL;
  const int block = 256;
  int64_t blocks = (nch + block - 1) / block;
  const int64_t cap = 256 * 16;  // 16 workgroups per CU, grid-stride beyond
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  if (!absmax_ready) {
    hipLaunchKernelGGL(fill_u32_kernel, dim3(2), dim3(256), 0, st, (uint32_t*)absmax, 0u, (int)(STAT_SLOT_BYTES / 4));
    hipLaunchKernelGGL((hq_absmax_kernel<T, N>), dim3((unsigned)blocks), dim3(block), 0, st, (const T*)in, nch, absmax, nrt);
  }
  hipLaunchKernelGGL((hq_tensor_kernel<T, N, BITS, ROUND>), dim3((unsigned)blocks), dim3(block), 0, st,
                     (const T*)in, nch, K / EPL, ld, absmax, (int8_t*)codes, scales, seed, stream_id, nrt);
  return check_launch("hq_tensor_kernel");
}

template <typename T, int N, int BITS, int ROUND>
static int launch_groups(const void* in, int64_t M, int64_t K, void* codes, int64_t ld, float* scales, float* gmax,
                         float* group_steps, int64_t group_rows, uint64_t seed, uint32_t stream_id, hipStream_t st, int nrt) {
  const int64_t groups = M / group_rows, cpg = group_rows * (K / EPL);
  int64_t bx = (cpg + 255) / 256;
  const int64_t cap = (256 * 16 + groups - 1) / groups;    // about 16 workgroups per CU in all
  if (bx > cap) bx = cap;
  if (bx < 1) bx = 1;
  if (groups > 65535) return fail(HOT_ERR_UNSUPPORTED, "hot_hq_rowwise: more than 65535 sample groups");
  const dim3 grid((unsigned)bx, (unsigned)groups);
  hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((groups * GROUP_STAT_STRIDE + 255) / 256)), dim3(256), 0, st, (uint32_t*)gmax, 0u, (int)(groups * GROUP_STAT_STRIDE));
  hipLaunchKernelGGL((hq_group_absmax_kernel<T, N>), grid, dim3(256), 0, st, (const T*)in, cpg, gmax, nrt);
  hipLaunchKernelGGL((hq_group_quant_kernel<T, N, BITS, ROUND>), grid, dim3(256), 0, st, (const T*)in, cpg, K / EPL, ld, gmax,
                     (int8_t*)codes, scales, group_steps, seed, stream_id, nrt);
  return check_launch("hq_group_quant_kernel");
}

template <typename T, int N, int BITS, int ROUND>
static int dispatch_mode(int scale_mode, const void* in, int64_t M, int64_t K, void* codes, int64_t ld, float* scales,
                         float* absmax, uint64_t seed, uint32_t stream_id, hipStream_t st, bool absmax_ready, int nrt,
                         int64_t group_rows, float* group_steps) {
  const int64_t row_bytes = K * BITS / 8;
  if (ld > row_bytes) {
    const int64_t n = M * ((ld - row_bytes) / 4);
    hipLaunchKernelGGL(zero_pad_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (int8_t*)codes, M, row_bytes, ld);
  }
  if (scale_mode == HOT_SCALE_TENSOR && group_rows > 0)
    return launch_groups<T, N, BITS, ROUND>(in, M, K, codes, ld, scales, absmax, group_steps, group_rows, seed, stream_id, st, nrt);
  if (scale_mode == HOT_SCALE_ROW) return launch_row<T, N, BITS, ROUND>(in, M, K, codes, ld, scales, seed, stream_id, st, nrt);
  return launch_tensor<T, N, BITS, ROUND>(in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, nrt);
}

template <typename T, int N>
static int dispatch_bits(int bits, int rounding, int scale_mode, const void* in, int64_t M, int64_t K,
                         void* codes, int64_t ld, float* scales, float* absmax, uint64_t seed, uint32_t stream_id,
                         hipStream_t st, bool absmax_ready, int nrt, int64_t group_rows, float* group_steps) {
  if (bits == 4) {
    return rounding == HOT_ROUND_NEAREST
               ? dispatch_mode<T, N, 4, 0>(scale_mode, in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, nrt, group_rows, group_steps)
               : dispatch_mode<T, N, 4, 1>(scale_mode, in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, nrt, group_rows, group_steps);
  }
  return rounding == HOT_ROUND_NEAREST
             ? dispatch_mode<T, N, 8, 0>(scale_mode, in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, nrt, group_rows, group_steps)
             : dispatch_mode<T, N, 8, 1>(scale_mode, in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, nrt, group_rows, group_steps);
}

template <typename T>
static int dispatch_n(int n, int bits, int rounding, int scale_mode, const void* in, int64_t M, int64_t K,
                      void* codes, int64_t ld, float* scales, float* absmax, uint64_t seed, uint32_t stream_id,
                      hipStream_t st, bool absmax_ready, int64_t group_rows, float* group_steps) {
  switch (n) {
    case 1: case 2: case 4: case 8:
      return dispatch_bits<T, 8>(bits, rounding, scale_mode, in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, n, group_rows, group_steps);
    case 16: return dispatch_bits<T, 16>(bits, rounding, scale_mode, in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, n, group_rows, group_steps);
    case 32: return dispatch_bits<T, 32>(bits, rounding, scale_mode, in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, n, group_rows, group_steps);
    default: return dispatch_bits<T, 64>(bits, rounding, scale_mode, in, M, K, codes, ld, scales, absmax, seed, stream_id, st, absmax_ready, n, group_rows, group_steps);
  }
}

template <typename T, int N>
static int launch_luq(const void* in, int64_t M, int64_t K, int bits, void* codes, int64_t ld, int64_t kp, float* scale,
                      float* slots, uint64_t seed, uint32_t rng_stream, hipStream_t st, int nrt) {
  const int64_t nch = M * K / EPL;
  int64_t blocks = (nch + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  if (blocks < 1) blocks = 1;
  const int lev = (1 << (bits - 1)) - 1;
  hipLaunchKernelGGL(fill_u32_kernel, dim3(2), dim3(256), 0, st, (uint32_t*)slots, 0u, (int)(STAT_SLOT_BYTES / 4));
  hipLaunchKernelGGL((hq_posmax_kernel<T, N>), dim3((unsigned)blocks), dim3(256), 0, st, (const T*)in, nch, slots, nrt);
  hipLaunchKernelGGL((hq_luq_kernel<T, N>), dim3((unsigned)blocks), dim3(256), 0, st, (const T*)in, nch, K / EPL, ld, kp,
                     slots, 1.0f / (float)(1 << lev), (int8_t*)codes, scale, seed, rng_stream, nrt);
  return check_launch("hq_luq_kernel");
}

template <typename T>
static int dispatch_luq(int n, const void* in, int64_t M, int64_t K, int bits, void* codes, int64_t ld, int64_t kp,
                        float* scale, float* slots, uint64_t seed, uint32_t rng_stream, hipStream_t st) {
  switch (n) {
    case 1: case 2: case 4: case 8: return launch_luq<T, 8>(in, M, K, bits, codes, ld, kp, scale, slots, seed, rng_stream, st, n);
    case 16: return launch_luq<T, 16>(in, M, K, bits, codes, ld, kp, scale, slots, seed, rng_stream, st, n);
    case 32: return launch_luq<T, 32>(in, M, K, bits, codes, ld, kp, scale, slots, seed, rng_stream, st, n);
    default: return launch_luq<T, 64>(in, M, K, bits, codes, ld, kp, scale, slots, seed, rng_stream, st, n);
  }
}

int hq_luq_impl(const void* in, int dtype, int64_t M, int64_t K, int n, int bits, uint64_t seed, void* codes_out,
                int64_t kp, float* scale_out, void* workspace, size_t workspace_bytes, hipStream_t st, uint32_t rng_stream) {
  const char* who = "hq_luq";
  if (!in || !codes_out || !scale_out) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (M <= 0 || K <= 0 || K % 8) return fail(HOT_ERR_INVALID, "%s: bad shape M=%lld K=%lld (K a multiple of 8)", who, (long long)M, (long long)K);
  if (n < 1 || n > 64 || (n & (n - 1)) || K % n) return fail(HOT_ERR_UNSUPPORTED, "%s: Hadamard block %d (a power of two up to 64 dividing K)", who, n);
  if (bits != 4) return fail(HOT_ERR_UNSUPPORTED, "%s: bits=%d (the two-plane code layout is sized for 4)", who, bits);
  if (kp < K || (kp & 15)) return fail(HOT_ERR_INVALID, "%s: plane width %lld must be a multiple of 16 and >= K", who, (long long)kp);
  if (!workspace || workspace_bytes < STAT_SLOT_BYTES) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed", who, STAT_SLOT_BYTES);
  if (((uintptr_t)in & 15) || ((uintptr_t)codes_out & 15)) return fail(HOT_ERR_INVALID, "%s: pointers must be 16-byte aligned", who);
  // bytes [K, 2 kp) of every row first: the K padding of both planes (the second plane is written afterwards)
  zero_pad_impl(codes_out, M, K, 2 * kp, st);
  float* slots = (float*)workspace;
  switch (dtype) {
    case HOT_F32: return dispatch_luq<float>(n, in, M, K, bits, codes_out, 2 * kp, kp, scale_out, slots, seed, rng_stream, st);
    case HOT_BF16: return dispatch_luq<bf16_t>(n, in, M, K, bits, codes_out, 2 * kp, kp, scale_out, slots, seed, rng_stream, st);
    case HOT_F16: return dispatch_luq<f16_t>(n, in, M, K, bits, codes_out, 2 * kp, kp, scale_out, slots, seed, rng_stream, st);
    default: return fail(HOT_ERR_INVALID, "%s: bad dtype %d", who, dtype);
  }
}

int luq_pair_impl(const void* qw, int64_t rows, int64_t kp, void* out, hipStream_t st) {
  if (!qw || !out || rows <= 0 || kp <= 0 || (kp & 15)) return fail(HOT_ERR_INVALID, "luq_pair: bad arguments");
  const int64_t n = rows * (kp / 16);
  hipLaunchKernelGGL(luq_pair_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (const int8_t*)qw, rows, kp, (int8_t*)out);
  return check_launch("luq_pair_kernel");
}

int hq_rowwise_impl(const void* in, int dtype, int64_t M, int64_t K, int n, int bits, int rounding,
                    uint64_t seed, uint32_t rng_stream, int scale_mode, void* codes_out, int64_t ld_codes,
                    float* scales_out, void* workspace, size_t workspace_bytes, hipStream_t st, bool absmax_ready,
                    int64_t group_rows, float* group_steps) {
  if (M != 0 && (!in || !codes_out || !scales_out)) return fail(HOT_ERR_INVALID, "hot_hq_rowwise: null pointer");
  if (M < 0 || K <= 0) return fail(HOT_ERR_INVALID, "hot_hq_rowwise: bad shape M=%lld K=%lld", (long long)M, (long long)K);
  if (n < 1 || n > 64 || (n & (n - 1))) return fail(HOT_ERR_UNSUPPORTED, "hot_hq_rowwise: Hadamard block %d (a power of two up to 64)", n);
  if (K % n || K % 8) return fail(HOT_ERR_INVALID, "hot_hq_rowwise: K=%lld is not a multiple of the block %d and of 8", (long long)K, n);
  if (bits != 4 && bits != 8) return fail(HOT_ERR_UNSUPPORTED, "hot_hq_rowwise: bits=%d (4 or 8)", bits);
  if (rounding != HOT_ROUND_NEAREST && rounding != HOT_ROUND_STOCH) return fail(HOT_ERR_INVALID, "hot_hq_rowwise: bad rounding %d", rounding);
  if (scale_mode != HOT_SCALE_TENSOR && scale_mode != HOT_SCALE_ROW) return fail(HOT_ERR_UNSUPPORTED, "hot_hq_rowwise: scale mode %d (tensor or row)", scale_mode);
  if (((uintptr_t)in & 15) || ((uintptr_t)codes_out & 7)) return fail(HOT_ERR_INVALID, "hot_hq_rowwise: input must be 16-byte and output 8-byte aligned");
  if (M >= (1ll << 31)) return fail(HOT_ERR_UNSUPPORTED, "hot_hq_rowwise: M too large");
  if (ld_codes < K * bits / 8 || (ld_codes & 7)) return fail(HOT_ERR_INVALID, "hot_hq_rowwise: code pitch %lld must be a multiple of 8 and >= %lld", (long long)ld_codes, (long long)(K * bits / 8));
  float* absmax = nullptr;
  if (group_rows < 0 || (group_rows > 0 && (M % group_rows || scale_mode != HOT_SCALE_TENSOR)))
    return fail(HOT_ERR_INVALID, "hot_hq_rowwise: %lld rows are not whole groups of %lld rows with one step each", (long long)M, (long long)group_rows);
  if (scale_mode == HOT_SCALE_TENSOR) {
    const size_t need = group_rows > 0 ? (size_t)(M / group_rows) * 128 : STAT_SLOT_BYTES;
    if (!workspace || workspace_bytes < need) return fail(HOT_ERR_WORKSPACE, "hot_hq_rowwise: per-tensor scale needs a %zu-byte workspace", need);
    absmax = (float*)workspace;
  }
  if (M == 0) return HOT_OK;
  switch (dtype) {
    case HOT_F32: return dispatch_n<float>(n, bits, rounding, scale_mode, in, M, K, codes_out, ld_codes, scales_out, absmax, seed, rng_stream, st, absmax_ready, group_rows, group_steps);
    case HOT_BF16: return dispatch_n<bf16_t>(n, bits, rounding, scale_mode, in, M, K, codes_out, ld_codes, scales_out, absmax, seed, rng_stream, st, absmax_ready, group_rows, group_steps);
    case HOT_F16: return dispatch_n<f16_t>(n, bits, rounding, scale_mode, in, M, K, codes_out, ld_codes, scales_out, absmax, seed, rng_stream, st, absmax_ready, group_rows, group_steps);
    default: return fail(HOT_ERR_INVALID, "hot_hq_rowwise: bad dtype %d", dtype);
  }
}

}  // namespace hot
