// Hadamard low-rank projection along tokens for blocks larger than one thread can hold:
// n = 64 m tokens, m = 4 .. 128 (the reference's make_WHT rule asks for the largest power of two
// dividing the token count, e.g. 8192 for 8192 tokens; utils/hadamard_matmul.py:209-226).  Blocks of
// up to 128 tokens are served by the register kernel (colwise.hip).
//
// A Sylvester transform of n = 64 m points is the 64-point transform inside each run of 64 rows
// followed by the m-point transform across the runs, and the canonical butterfly order
// (h = 1, 2, 4, ...) is exactly that sequence: stages h < 64 stay inside a run, stages h >= 64 pair
// run j with run j ^ (h / 64).  Two kernels therefore reproduce the one-pass arithmetic bit for bit:
//   stage 1   every run of 64 rows of a channel -> fp32 coefficients, written back in place of the
//             rows into a workspace T [R, C]
//   stage 2   for coefficient k of the runs of one block: the m values T[(64 j + k), c] -> m-point
//             transform -> natural-order coefficient 64 j + k of the block; kept ones are measured
//             (statistics pass) or quantised (quantise pass) into codes [L', C]
//   transpose codes [L', C] -> [C, ld] (K-major for the GEMM), padding zeroed
// Only the coefficients a kept row needs make the round trip: natural row i of a block is coefficient
// k = i % 64 of run i / 64, so a k that no kept row has is never written by stage 1 nor read by stage 2
// (the make_WHT selections keep no odd row: half the traffic).  The row table lives in the workspace
// and is written by kernels whose arguments carry the rows by value, so the whole call is a sequence
// of launches: no host-to-device copy, nothing read from host memory after the call returns, and a
// stream under graph capture records it like any other call.
// This is the exactness path for large blocks, not a tuned one: the input is read with scalar loads
// and the coefficients make a round trip through HBM in fp32.
#include <string.h>

#include <algorithm>
#include <memory>

#include "hot_device.h"
#include "hot_host.h"

namespace hot {

namespace {

constexpr int BT = 256;  // threads per workgroup = channels per workgroup
constexpr size_t STAT_BYTES = 256 + STAT_SLOT_BYTES;   // [0] absmax, [1] step, [2] clip; then the absmax slots

struct BigArgs {
  const void* in;
  float* T;            // [R, C] fp32 coefficients of the 64-point stage
  int8_t* tmp;         // [Kout, tmp_ld] codes before the transpose (or the untransposed destination itself)
  int64_t tmp_ld;
  const int32_t* tab;  // per natural row of a block: slot | visit << 16, or -1 when dropped
  int64_t R, C, NB;    // NB = R / n blocks
  int32_t n, r, rpad, bits, rounding, mode;
  int32_t nk;          // coefficients of a 64-run that some kept row needs
  uint64_t kmask;      // bit k: coefficient k is one of them
  uint8_t klist[64];   // the nk set bits of kmask in increasing order
  // run-major row lists only (big_stage2_runs_kernel): which runs keep needed coefficient index kc
  // (bit j of keep[kc]: natural row 64 j + klist[kc] is kept), and the output coefficient of its first
  // kept row (kbase[kc]; kbase[nk] = r): its other kept rows follow in run order
  uint32_t keep[64][4];
  uint16_t kbase[65];
  float* stat;         // [0] absmax, [1] step, [2] clip; the absmax slots from word 64
  float* colmax;       // per-channel absmax (ROW)
  double* partial;     // SAWB: 2 doubles per workgroup
  float* scales_out;
  float* row_absmax;   // stage 1 with RS: absmax of the row-wise 16-point Hadamard (STAT_SLOTS partial maxima), or null
  uint64_t seed;
  uint32_t stream;
};

template <typename T> __device__ __forceinline__ float load_f32(const T* p);
template <> __device__ __forceinline__ float load_f32<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p) { return as_f((uint32_t)p->v << 16); }
template <> __device__ __forceinline__ float load_f32<f16_t>(const f16_t* p) { return (float)p->v; }

template <int N>
__device__ __forceinline__ void fwht(float (&v)[N]) {
#pragma unroll
  for (int h = 1; h < N; h <<= 1) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if ((i & h) == 0) {
        const float a = v[i], b = v[i + h];
        v[i] = a + b;
        v[i + h] = a - b;
      }
    }
  }
}

// RS: the pass also tracks the absmax of the ROW-wise 16-point block Hadamard of the same input (the
// statistic of the row-wise quantiser of g_y, so that g_y is not read a further time for it).
// Adjacent lanes hold adjacent channels; within each group of 16 lanes the channels are dealt out so
// that the four stages of the 16-point transform pair lanes at the distances a single DPP operand
// reaches (channel bit 0 <-> lane xor 1, bit 1 <-> xor 2, bit 2 <-> xor 15, bit 3 <-> xor 8).  A stage
// computes own + s * partner with s = -1 on the lane of the upper channel of a pair: a lane's value
// may come out negated, magnitudes are those of the add / sub butterflies (the product with +-1 is
// exact).  C must be a multiple of 16: a group of 16 lanes is whole or absent.
template <typename T, bool RS>
__global__ void __launch_bounds__(BT) big_stage1_kernel(const BigArgs a) {
  __shared__ float s_max[BT / 64];
  const int tid = threadIdx.x;
  const int chan = RS ? (tid ^ ((tid & 4) ? 0xB : 0)) : tid;
  const int64_t c = (int64_t)blockIdx.x * BT + chan;
  const bool active = c < a.C;
  if (!RS && !active) return;
  const int64_t row0 = (int64_t)blockIdx.y * 64;
  const T* in = reinterpret_cast<const T*>(a.in) + row0 * a.C + (active ? c : 0);
  float v[64];
#pragma unroll
  for (int i = 0; i < 64; ++i) v[i] = load_f32<T>(in + (int64_t)i * a.C);
  if constexpr (RS) {
    const float sg1 = (chan & 1) ? -1.f : 1.f, sg2 = (chan & 2) ? -1.f : 1.f;
    const float sg4 = (chan & 4) ? -1.f : 1.f, sg8 = (chan & 8) ? -1.f : 1.f;
    float rmax = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float t[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) t[i] = v[16 * g + i];
      // every row is in its register before the first DPP read (the compiler's hazard check does not
      // look into asm statements); the stages run row-major over the sixteen rows, so no DPP read
      // follows the write of its register within two instructions
      asm volatile("s_nop 1"
                   : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]), "+v"(t[7]),
                     "+v"(t[8]), "+v"(t[9]), "+v"(t[10]), "+v"(t[11]), "+v"(t[12]), "+v"(t[13]), "+v"(t[14]), "+v"(t[15]));
#pragma unroll
      for (int i = 0; i < 16; ++i)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "+v"(t[i]) : "v"(sg1));
#pragma unroll
      for (int i = 0; i < 16; ++i)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "+v"(t[i]) : "v"(sg2));
#pragma unroll
      for (int i = 0; i < 16; ++i)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 row_mirror row_mask:0xf bank_mask:0xf" : "+v"(t[i]) : "v"(sg4));
#pragma unroll
      for (int i = 0; i < 16; ++i)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 row_ror:8 row_mask:0xf bank_mask:0xf" : "+v"(t[i]) : "v"(sg8));
#pragma unroll
      for (int i = 0; i < 16; ++i) rmax = fmaxf(rmax, fabsf(t[i]));
    }
    const float m = wave_max(active ? rmax : 0.f);
    if ((tid & 63) == 0) s_max[tid >> 6] = m;
    __syncthreads();
    if (tid == 0) {
      float mm = s_max[0];
      for (int i = 1; i < BT / 64; ++i) mm = fmaxf(mm, s_max[i]);
      stat_slot_update(a.row_absmax, blockIdx.y * gridDim.x + blockIdx.x, mm);
    }
    if (!active) return;
  }
  fwht<64>(v);
  float* out = a.T + (int64_t)blockIdx.y * a.nk * a.C + c;    // T [run][needed coefficient][channel]
#pragma unroll
  for (int i = 0; i < 64; ++i)
    if ((a.kmask >> i) & 1ull) { *out = v[i]; out += a.C; }
}

// the 16-bit uniform integer of element e
__device__ __forceinline__ uint32_t bits_of(uint64_t e, uint64_t seed, uint32_t stream) {
  return sr_bits_of(sr_octet_words(e >> 3, seed, stream), (uint32_t)e);
}

// blockIdx.y = block * nk + (index of k among the needed coefficients)
template <int M, int PASS, int ROUND, bool SAWB>
__global__ void __launch_bounds__(BT) big_stage2_kernel(const BigArgs a) {
  __shared__ float s_max[BT / 64];
  __shared__ double s_sum[2][BT / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t c = (int64_t)blockIdx.x * BT + tid;
  const bool active = c < a.C;
  const int64_t blk = blockIdx.y / a.nk;
  const int kc = (int)(blockIdx.y - blk * a.nk);
  const int k = a.klist[kc];
  const int qmax = (1 << (a.bits - 1)) - 1;
  // The table entries of this coefficient index (one per run) go through LDS: read from global memory
  // inside the quantise loop they would sit between the loop's byte stores, and every such load then
  // waits for the store before it (one memory round trip per kept row).
  __shared__ int32_t s_tab[M];
  if (tid < M) s_tab[tid] = a.tab[tid * 64 + k];
  __syncthreads();
  float v[M];
  if (active) {
    const float* t = a.T + ((blk * M) * a.nk + kc) * a.C + c;
#pragma unroll
    for (int j = 0; j < M; ++j) v[j] = t[(int64_t)j * a.nk * a.C];
  } else {
#pragma unroll
    for (int j = 0; j < M; ++j) v[j] = 0.f;
  }
  fwht<M>(v);
  // every coefficient is complete here: without this the compiler sinks the last butterfly stage into
  // the conditional code below and holds both stages' registers (a third more than the block itself)
  if constexpr (PASS == 1 || SAWB) {
#pragma unroll
    for (int j = 0; j < M; ++j) asm volatile("" : "+v"(v[j]));
  }

  if constexpr (PASS == 0) {
    float cmax = 0.f;
    double ssq = 0.0, sab = 0.0;
#pragma unroll
    for (int j = 0; j < M; ++j) {
      if (s_tab[j] >= 0) {
        cmax = fmaxf(cmax, fabsf(v[j]));
        if constexpr (SAWB) { ssq += (double)v[j] * (double)v[j]; sab += (double)fabsf(v[j]); }
      }
    }
    if (a.mode == HOT_SCALE_ROW) {
      if (active) atomic_max_nonneg(a.colmax + c, cmax);
      return;
    }
    if (a.mode == HOT_SCALE_TENSOR) {
      const float m = wave_max(active ? cmax : 0.f);
      if (lane == 0) s_max[wave] = m;
      __syncthreads();
      if (tid == 0) {
        float mm = s_max[0];
        for (int i = 1; i < BT / 64; ++i) mm = fmaxf(mm, s_max[i]);
        stat_slot_update(a.stat + 64, blockIdx.y * gridDim.x + blockIdx.x, mm);
      }
      return;
    }
    ssq = wave_sum(active ? ssq : 0.0);
    sab = wave_sum(active ? sab : 0.0);
    if (lane == 0) { s_sum[0][wave] = ssq; s_sum[1][wave] = sab; }
    __syncthreads();
    if (tid == 0) {
      double q = 0.0, b = 0.0;
      for (int i = 0; i < BT / 64; ++i) { q += s_sum[0][i]; b += s_sum[1][i]; }
      const int64_t wg = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
      a.partial[2 * wg] = q;
      a.partial[2 * wg + 1] = b;
    }
  } else {
    if (!active) return;
    float d, clip = 0.f;
    if (a.mode == HOT_SCALE_ROW) d = a.colmax[c] / (float)qmax + 1e-11f;
    else if (a.mode == HOT_SCALE_TENSOR) d = a.stat[0] / (float)qmax + 1e-11f;
    else { d = a.stat[1] + 1e-11f; clip = a.stat[2]; }
    const float rcp = 1.0f / d;
#pragma unroll
    for (int j = 0; j < M; ++j) {
      const int32_t e = s_tab[j];
      if (e < 0) continue;
      const int slot = e & 0xFFFF, visit = e >> 16;
      float x = v[j];
      if constexpr (SAWB) x = fminf(fmaxf(x, -clip), clip);
      int q;
      if constexpr (ROUND == HOT_ROUND_NEAREST) {
        q = (int)rint_div_fast(x, d, rcp);      // bit for bit rintf(x / d)
      } else {
        const uint64_t idx = ((uint64_t)c * (uint64_t)a.NB + (uint64_t)blk) * (uint64_t)a.rpad + (uint64_t)visit;
        q = q_stoch_fix(x, rcp * 65536.0f, bits_of(idx, a.seed, a.stream), qmax);
      }
      a.tmp[(blk * a.r + slot) * a.tmp_ld + c] = (int8_t)q;
    }
  }
}

// Quantise pass for row lists in "run-major" order: the kept rows sorted by (row % 64, row / 64).  The
// order of the kept coefficients along K is the caller's (slot = position in its list) and means
// nothing to the product that consumes them, as long as both operands use the same; in this order
// the coefficients that one coefficient index k of the 64-point stage yields -- what a thread of
// this pass computes -- are neighbours along K, so a workgroup (64 channels x KG consecutive
// needed indices, one per wave) owns ONE contiguous K run of every channel: the codes are staged
// in LDS as [channel][run] and leave K-major, straight into the GEMM operand.  No [K, C]
// intermediate with its 64-byte stores, no transpose kernel.  The workgroup of a block's last
// index group also clears the row padding behind the last block.
constexpr int KG = 4;
template <int M, int ROUND, bool SAWB>
__global__ void __launch_bounds__(64 * KG, 2) big_stage2_runs_kernel(const BigArgs a, int8_t* __restrict__ out, int64_t ld_out, int groups) {
  __shared__ __align__(16) uint8_t img[64][KG * M + 16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t c0 = (int64_t)blockIdx.x * 64, c = c0 + lane;
  const bool active = c < a.C;
  const int64_t blk = blockIdx.y / groups;
  const int grp = (int)(blockIdx.y - blk * groups);
  const int kc = grp * KG + wave;                      // this wave's needed coefficient index
  const bool has_k = kc < a.nk;
  const int qmax = (1 << (a.bits - 1)) - 1;
  // the workgroup's K run within the block: the outputs of its coefficient indices, in list order
  const int k_hi = (grp + 1) * KG < a.nk ? (grp + 1) * KG : a.nk;
  const int run0 = a.kbase[grp * KG], run_len = a.kbase[k_hi] - run0;
  // absmax steps come straight from the statistic (no finalize kernel in between); the workgroups of
  // the first block and index group publish them
  float d = 1.f, clip = 0.f;
  if (a.mode == HOT_SCALE_ROW) {
    const float sc = (active ? a.colmax[c] : 0.f) / (float)qmax;
    d = sc + 1e-11f;
    if (active && blockIdx.y == 0 && wave == 0) a.scales_out[c] = sc;
  } else if (a.mode == HOT_SCALE_TENSOR) {
    const float sc = stat_slots_max(a.stat + 64, lane) / (float)qmax;
    d = sc + 1e-11f;
    if (blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) a.scales_out[0] = sc;
  } else {
    d = a.stat[1] + 1e-11f;
    clip = a.stat[2];
  }
  const float rcp = 1.0f / d;
  if (has_k) {
    float v[M];
    if (active) {
      const float* t = a.T + ((blk * M) * a.nk + kc) * a.C + c;
#pragma unroll
      for (int j = 0; j < M; ++j) v[j] = t[(int64_t)j * a.nk * a.C];
    } else {
#pragma unroll
      for (int j = 0; j < M; ++j) v[j] = 0.f;
    }
    fwht<M>(v);
    // every coefficient is complete here: without this the compiler sinks the last butterfly stage into
    // the conditional code below and holds both stages' registers (a third more than the block itself)
#pragma unroll
    for (int j = 0; j < M; ++j) asm volatile("" : "+v"(v[j]));
    // which runs keep this coefficient index: a bit mask in the kernel arguments, the same for every
    // lane of the wave, so the walk below branches on scalar registers and a kept coefficient's place
    // in the run is a running count (the list is run-major: this index's outputs are neighbours)
    const int k = a.klist[kc];
    int pos = __builtin_amdgcn_readfirstlane((int)a.kbase[kc] - run0);
    uint32_t kw[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) kw[w] = __builtin_amdgcn_readfirstlane(a.keep[kc][w]);
#pragma unroll
    for (int j = 0; j < M; ++j) {
      if (!((kw[j >> 5] >> (j & 31)) & 1u)) continue;
      float x = v[j];
      if constexpr (SAWB) x = fminf(fmaxf(x, -clip), clip);
      int q;
      if constexpr (ROUND == HOT_ROUND_NEAREST) {
        q = (int)rint_div_fast(x, d, rcp);      // bit for bit rintf(x / d)
      } else {
        const int visit = a.tab[j * 64 + k] >> 16;
        const uint64_t idx = ((uint64_t)c * (uint64_t)a.NB + (uint64_t)blk) * (uint64_t)a.rpad + (uint64_t)visit;
        q = q_stoch_fix(x, rcp * 65536.0f, bits_of(idx, a.seed, a.stream), qmax);
      }
      img[lane][pos++] = (uint8_t)(q & 0xFF);
    }
  }
  __syncthreads();
  // flush: bytes [blk r + run0, + run_len) of every channel's row, dword by dword on the dwords of
  // the destination (its first and last dword may belong to the run only in part)
  const int nch = (int)((a.C - c0) < 64 ? (a.C - c0) : 64);
  if (run_len > 0) {
    const int64_t b0 = blk * a.r + run0, b1 = b0 + run_len;          // byte range within the row
    const int64_t w0 = b0 >> 2, w1 = (b1 + 3) >> 2;                  // destination dwords [w0, w1)
    const int nw = (int)(w1 - w0);
    for (int i = tid; i < nch * nw; i += 64 * KG) {
      const int rch = i / nw;
      const int64_t w = w0 + (i - rch * nw);
      int8_t* dst = out + (c0 + rch) * ld_out + w * 4;
      const int off = (int)(w * 4 - b0);                              // position of the dword's first byte in the run
      if (off >= 0 && off + 4 <= run_len) {
        const uint8_t* src = &img[rch][off];
        const uint32_t word = (uint32_t)src[0] | ((uint32_t)src[1] << 8) | ((uint32_t)src[2] << 16) | ((uint32_t)src[3] << 24);
        *reinterpret_cast<uint32_t*>(dst) = word;
      } else {
#pragma unroll
        for (int t = 0; t < 4; ++t)
          if (off + t >= 0 && off + t < run_len) dst[t] = (int8_t)img[rch][off + t];
      }
    }
  }
  if (blk == a.NB - 1 && grp == groups - 1) {
    const int64_t k_end = a.NB * a.r;
    const int pad = (int)(ld_out - k_end);
    for (int i = tid; i < nch * pad; i += 64 * KG) {
      const int rch = i / pad;
      out[(c0 + rch) * ld_out + k_end + (i - rch * pad)] = 0;
    }
  }
}

template <int M>
int launch_runs(const BigArgs& a, void* out, int64_t ld_out, hipStream_t st) {
  const int groups = (a.nk + KG - 1) / KG;
  const dim3 grid((unsigned)((a.C + 63) / 64), (unsigned)(a.NB * groups));
  const bool sawb = a.mode == HOT_SCALE_SAWB, stoch = a.rounding == HOT_ROUND_STOCH;
  if (stoch) {
    if (sawb) hipLaunchKernelGGL((big_stage2_runs_kernel<M, 1, true>), grid, dim3(64 * KG), 0, st, a, (int8_t*)out, ld_out, groups);
    else hipLaunchKernelGGL((big_stage2_runs_kernel<M, 1, false>), grid, dim3(64 * KG), 0, st, a, (int8_t*)out, ld_out, groups);
  } else {
    if (sawb) hipLaunchKernelGGL((big_stage2_runs_kernel<M, 0, true>), grid, dim3(64 * KG), 0, st, a, (int8_t*)out, ld_out, groups);
    else hipLaunchKernelGGL((big_stage2_runs_kernel<M, 0, false>), grid, dim3(64 * KG), 0, st, a, (int8_t*)out, ld_out, groups);
  }
  return check_launch("big_stage2_runs_kernel");
}

int dispatch_runs(int m, const BigArgs& a, void* out, int64_t ld_out, hipStream_t st) {
  switch (m) {
    case 4: return launch_runs<4>(a, out, ld_out, st);
    case 8: return launch_runs<8>(a, out, ld_out, st);
    case 16: return launch_runs<16>(a, out, ld_out, st);
    case 32: return launch_runs<32>(a, out, ld_out, st);
    case 64: return launch_runs<64>(a, out, ld_out, st);
    case 128: return launch_runs<128>(a, out, ld_out, st);
    default: return fail(HOT_ERR_UNSUPPORTED, "hla: block size %d (64 m with m a power of two, 4 .. 128)", 64 * m);
  }
}

__global__ void big_clear_kernel(float* stat, float* colmax, int64_t C, int32_t* tab, int n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < (int64_t)(STAT_BYTES / 4)) stat[i] = 0.f;
  if (i < C) colmax[i] = 0.f;
  if (i < n) tab[i] = -1;
}

// The row table, built by ONE launch whose arguments carry the kept rows by value: up to 2304 rows
// of 13 bits each (3744 bytes of the 4 KiB a launch may carry; larger selections go in pieces of that
// size).  Entry of natural row i: its output coefficient (the position of i in the caller's list) in
// the low half, its visit number (the rank of i among the kept rows in natural order, which numbers
// the elements of stochastic rounding) in the high half; -1 for dropped rows (written by the clear
// kernel).  The rank is counted on the device: thread k compares its row with every row of the call.
constexpr int TAB_ROWS = 2304;
struct TabRows { uint32_t packed[(TAB_ROWS * 13 + 31) / 32]; int32_t count; };
__device__ __host__ inline int tab_row_get(const uint32_t* packed, int i) {
  const int bit = i * 13, w = bit >> 5, sh = bit & 31;
  uint32_t v = packed[w] >> sh;
  if (sh > 19) v |= packed[w + 1] << (32 - sh);
  return (int)(v & 0x1FFFu);
}
inline void tab_row_put(uint32_t* packed, int i, int row) {
  const int bit = i * 13, w = bit >> 5, sh = bit & 31;
  packed[w] |= (uint32_t)row << sh;
  if (sh > 19) packed[w + 1] |= (uint32_t)row >> (32 - sh);
}
__global__ void __launch_bounds__(256) big_table_kernel(int32_t* tab, const TabRows p) {
  // every workgroup marks the kept rows in a bitmap of the block's n <= 8192 natural rows; the rank
  // of a row is the number of marks below it
  __shared__ uint32_t s_map[8192 / 32];
  __shared__ uint32_t s_below[8192 / 32];
  const int tid = threadIdx.x;
  s_map[tid] = 0u;
  __syncthreads();
  for (int j = tid; j < p.count; j += 256) {
    const int row = tab_row_get(p.packed, j);
    atomicOr(&s_map[row >> 5], 1u << (row & 31));
  }
  __syncthreads();
  {
    // marks in the words before word `tid` (256 words: a serial sum per thread is short)
    uint32_t acc = 0;
    for (int w = 0; w < tid; ++w) acc += (uint32_t)__popc(s_map[w]);
    s_below[tid] = acc;
  }
  __syncthreads();
  const int k = blockIdx.x * 256 + tid;
  if (k >= p.count) return;
  const int row = tab_row_get(p.packed, k);
  const int rank = (int)(s_below[row >> 5] + (uint32_t)__popc(s_map[row >> 5] & ((1u << (row & 31)) - 1u)));
  tab[row] = k | (rank << 16);
}
// Clear and table in one launch (selections of up to TAB_ROWS rows): every workgroup marks the kept
// rows in its own LDS bitmap; thread i of the grid clears word i of the statistics and of the
// per-channel maxima, writes -1 for natural row i when it is dropped, and the entry of the i-th row of
// the caller's list.  Dropped and kept rows are disjoint, so the two writes never meet.
__global__ void __launch_bounds__(256) big_prepare_kernel(float* stat, float* colmax, int64_t C, int32_t* tab, int n, const TabRows p) {
  __shared__ uint32_t s_map[8192 / 32];
  __shared__ uint32_t s_below[8192 / 32];
  const int tid = threadIdx.x;
  s_map[tid] = 0u;
  __syncthreads();
  for (int j = tid; j < p.count; j += 256) {
    const int row = tab_row_get(p.packed, j);
    atomicOr(&s_map[row >> 5], 1u << (row & 31));
  }
  __syncthreads();
  {
    uint32_t acc = 0;
    for (int w = 0; w < tid; ++w) acc += (uint32_t)__popc(s_map[w]);
    s_below[tid] = acc;
  }
  __syncthreads();
  const int64_t i = (int64_t)blockIdx.x * 256 + tid;
  if (i < (int64_t)(STAT_BYTES / 4)) stat[i] = 0.f;
  if (i < C) colmax[i] = 0.f;
  if (i < n && !((s_map[i >> 5] >> (i & 31)) & 1u)) tab[i] = -1;
  if (i < p.count) {
    const int row = tab_row_get(p.packed, (int)i);
    const int rank = (int)(s_below[row >> 5] + (uint32_t)__popc(s_map[row >> 5] & ((1u << (row & 31)) - 1u)));
    tab[row] = (int)i | (rank << 16);
  }
}
// selections of more than TAB_ROWS rows: the host ranks, the rows travel with their visit numbers
constexpr int TAB_PIECE = 512;
struct TabPiece { uint16_t row[TAB_PIECE], visit[TAB_PIECE], slot[TAB_PIECE]; int32_t count; };
__global__ void big_table_piece_kernel(int32_t* tab, const TabPiece p) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < p.count) tab[p.row[i]] = (int32_t)p.slot[i] | ((int32_t)p.visit[i] << 16);
}

// statistics -> steps (absmax modes are also read directly by the quantise pass)
__global__ void __launch_bounds__(256) big_finalize_kernel(const BigArgs a, int64_t nwg, int64_t kout) {
  __shared__ double s_q[256], s_b[256];
  const float qmax = (float)((1 << (a.bits - 1)) - 1);
  const int tid = threadIdx.x;
  if (a.mode == HOT_SCALE_ROW) {
    for (int64_t c = tid; c < a.C; c += 256) a.scales_out[c] = a.colmax[c] / qmax;
    return;
  }
  if (a.mode == HOT_SCALE_TENSOR) {
    const float mx = stat_slots_max(a.stat + 64, tid & 63);
    if (tid == 0) { a.stat[0] = mx; a.scales_out[0] = mx / qmax; }
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
    const double cnt = (double)kout * (double)a.C;
    const float clip = (float)(12.1 * sqrt(s_q[0] / cnt) - 12.2 * (s_b[0] / cnt));
    const float s = clip / qmax;
    a.stat[1] = s;
    a.stat[2] = clip;
    a.scales_out[0] = s;
  }
}

// tmp [K, C] -> out [C, ld] with the bytes [K, ld) of every row zeroed; 64 x 64 tiles through LDS
__global__ void __launch_bounds__(256) transpose_i8_kernel(const int8_t* __restrict__ tmp, int64_t K, int64_t C,
                                                           int8_t* __restrict__ out, int64_t ld) {
  __shared__ int8_t tile[64][65];
  const int64_t k0 = (int64_t)blockIdx.x * 64, c0 = (int64_t)blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int64_t k = k0 + i, c = c0 + tx;
    tile[i][tx] = (k < K && c < C) ? tmp[k * C + c] : (int8_t)0;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int64_t c = c0 + i, k = k0 + tx;
    if (c < C && k < ld) out[c * ld + k] = tile[tx][i];
  }
}

// two channels to a byte, the even channel in bits 3:0 (the untransposed packed-INT4 operand)
__global__ void __launch_bounds__(256) pack4_rows_kernel(const int8_t* __restrict__ tmp, int64_t K, int64_t C,
                                                         int8_t* __restrict__ out, int64_t ld) {
  const int64_t half = C / 2;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= K * half) return;
  const int64_t k = i / half, b = i - k * half;
  const int lo = tmp[k * C + 2 * b], hi = tmp[k * C + 2 * b + 1];
  out[k * ld + b] = (int8_t)((lo & 0xF) | ((hi & 0xF) << 4));
}

// ---- expansion P^T t of large blocks (the schemes that project g_y along the tokens for the g_x product,
// utils/quant_matmul.py:334-337) ---------------------------------------------------------------------
// H_n is symmetric, so P^T t = H_n z with z = the r coefficients at their natural rows and zeros
// elsewhere, through the canonical butterflies (stages h = 1, 2, ..., n / 2 on the natural row index):
// the stages below 64 act inside the runs of 64 consecutive rows (pass A, thread = channel, one run),
// the stages from 64 up across the runs at a fixed position (pass B, thread = channel, one position),
// with the fp32 intermediate [n, C] per block in the workspace.  Pass B scales by `post` (exact: 1 / n).
struct ExpandBigArgs {
  const float* t;      // [NB r, C]
  float* U;            // [NB n, C]
  void* out;           // [NB n, C]
  const int32_t* tab;  // per natural row: slot | visit << 16, or -1
  int64_t C;
  int32_t r, m;
  float post;
};

__global__ void __launch_bounds__(BT) expand_runs_kernel(const ExpandBigArgs a) {
  const int64_t c = (int64_t)blockIdx.x * BT + threadIdx.x;
  if (c >= a.C) return;
  const int64_t blk = blockIdx.y / a.m;
  const int j = (int)(blockIdx.y - blk * a.m);
  float v[64];
#pragma unroll
  for (int k = 0; k < 64; ++k) {
    const int32_t e = a.tab[j * 64 + k];               // the same for every thread: a scalar load and branch
    v[k] = e >= 0 ? a.t[(blk * a.r + (e & 0xFFFF)) * a.C + c] : 0.f;
  }
  fwht<64>(v);
  float* u = a.U + ((blk * a.m + j) * 64) * a.C + c;
#pragma unroll
  for (int k = 0; k < 64; ++k) u[(int64_t)k * a.C] = v[k];
}

template <int M, typename OutT>
__global__ void __launch_bounds__(BT) expand_across_kernel(const ExpandBigArgs a) {
  const int64_t c = (int64_t)blockIdx.x * BT + threadIdx.x;
  if (c >= a.C) return;
  const int64_t blk = blockIdx.y / 64;
  const int k = (int)(blockIdx.y - blk * 64);
  const int64_t base = ((blk * M) * 64 + k) * a.C + c;
  float v[M];
#pragma unroll
  for (int j = 0; j < M; ++j) v[j] = a.U[base + (int64_t)j * 64 * a.C];
  fwht<M>(v);
  OutT* out = reinterpret_cast<OutT*>(a.out);
#pragma unroll
  for (int j = 0; j < M; ++j) store_scalar<OutT>(out + base + (int64_t)j * 64 * a.C, v[j] * a.post);
}

template <int M>
int launch_expand_across(const ExpandBigArgs& a, dim3 grid, int out_dtype, hipStream_t st) {
  switch (out_dtype) {
    case HOT_F32: hipLaunchKernelGGL((expand_across_kernel<M, float>), grid, dim3(BT), 0, st, a); break;
    case HOT_BF16: hipLaunchKernelGGL((expand_across_kernel<M, bf16_t>), grid, dim3(BT), 0, st, a); break;
    case HOT_F16: hipLaunchKernelGGL((expand_across_kernel<M, f16_t>), grid, dim3(BT), 0, st, a); break;
    default: return fail(HOT_ERR_INVALID, "hla_expand: bad out dtype %d", out_dtype);
  }
  return check_launch("expand_across_kernel");
}

__global__ void tab_clear_kernel(int32_t* tab, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) tab[i] = -1;
}

// Checks the row list and writes the table of a block (every entry: the clear kernel's -1 or a kept
// row's slot | visit << 16) with launches alone.
int build_row_table(int32_t* tab, int n, const int32_t* rows, int r, uint64_t* kmask_out, hipStream_t st, const char* who) {
  std::unique_ptr<int32_t[]> slot_of(new int32_t[(size_t)n]);
  for (int i = 0; i < n; ++i) slot_of[(size_t)i] = -1;
  uint64_t kmask = 0;
  for (int k = 0; k < r; ++k) {
    if (rows[k] < 0 || rows[k] >= n) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d outside [0, %d)", who, k, rows[k], n);
    if (slot_of[(size_t)rows[k]] != -1) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d listed twice", who, k, rows[k]);
    slot_of[(size_t)rows[k]] = k;
    kmask |= 1ull << (rows[k] & 63);
  }
  if (kmask_out) *kmask_out = kmask;
  if (r <= TAB_ROWS) {
    TabRows tr;
    memset(&tr, 0, sizeof(tr));
    tr.count = r;
    for (int k = 0; k < r; ++k) tab_row_put(tr.packed, k, rows[k]);
    hipLaunchKernelGGL(big_table_kernel, dim3((unsigned)((r + 255) / 256)), dim3(256), 0, st, tab, tr);
  } else {
    // rows in natural order: the visit number of a piece's entry i is its position in the sorted list
    std::unique_ptr<int32_t[]> sorted(new int32_t[(size_t)r]);
    for (int k = 0; k < r; ++k) sorted[(size_t)k] = rows[k];
    std::sort(sorted.get(), sorted.get() + r);
    for (int v0 = 0; v0 < r; v0 += TAB_PIECE) {
      TabPiece piece;
      piece.count = std::min(TAB_PIECE, r - v0);
      for (int i = 0; i < piece.count; ++i) {
        const int32_t row = sorted[(size_t)(v0 + i)];
        piece.row[i] = (uint16_t)row;
        piece.visit[i] = (uint16_t)(v0 + i);
        piece.slot[i] = (uint16_t)slot_of[(size_t)row];
      }
      hipLaunchKernelGGL(big_table_piece_kernel, dim3(TAB_PIECE / 256), dim3(256), 0, st, tab, piece);
    }
  }
  return check_launch("big_table_kernel");
}

template <int M>
int launch_stage2(const BigArgs& a, dim3 grid, int pass, hipStream_t st) {
  const bool sawb = a.mode == HOT_SCALE_SAWB, stoch = a.rounding == HOT_ROUND_STOCH;
  if (pass == 0) {
    if (sawb) hipLaunchKernelGGL((big_stage2_kernel<M, 0, 0, true>), grid, dim3(BT), 0, st, a);
    else hipLaunchKernelGGL((big_stage2_kernel<M, 0, 0, false>), grid, dim3(BT), 0, st, a);
  } else if (stoch) {
    if (sawb) hipLaunchKernelGGL((big_stage2_kernel<M, 1, 1, true>), grid, dim3(BT), 0, st, a);
    else hipLaunchKernelGGL((big_stage2_kernel<M, 1, 1, false>), grid, dim3(BT), 0, st, a);
  } else {
    if (sawb) hipLaunchKernelGGL((big_stage2_kernel<M, 1, 0, true>), grid, dim3(BT), 0, st, a);
    else hipLaunchKernelGGL((big_stage2_kernel<M, 1, 0, false>), grid, dim3(BT), 0, st, a);
  }
  return check_launch("big_stage2_kernel");
}

int dispatch_stage2(int m, const BigArgs& a, dim3 grid, int pass, hipStream_t st) {
  switch (m) {
    case 4: return launch_stage2<4>(a, grid, pass, st);
    case 8: return launch_stage2<8>(a, grid, pass, st);
    case 16: return launch_stage2<16>(a, grid, pass, st);
    case 32: return launch_stage2<32>(a, grid, pass, st);
    case 64: return launch_stage2<64>(a, grid, pass, st);
    case 128: return launch_stage2<128>(a, grid, pass, st);
    default: return fail(HOT_ERR_UNSUPPORTED, "hla: block size %d (64 m with m a power of two, 4 .. 128)", 64 * m);
  }
}


struct BigLayout { size_t off_colmax, off_partial, off_tab, off_T, off_tmp, total; };

BigLayout big_layout(int64_t R, int64_t C, int n, int r) {
  BigLayout b;
  size_t o = STAT_BYTES;
  b.off_colmax = o;  o += (size_t)round_up(C * 4, 256);
  b.off_partial = o; o += (size_t)(2 * sizeof(double)) * 65536;
  b.off_tab = o;     o += (size_t)round_up((int64_t)n * 4, 256);
  b.off_T = o;       o += (size_t)round_up(R * C * 4, 256);
  b.off_tmp = o;     o += (size_t)round_up((R / n) * r * C, 256);
  b.total = o;
  return b;
}

}  // namespace

size_t hla_big_workspace_bytes_impl(int64_t R, int64_t C, int n, int r) {
  if (R <= 0 || C <= 0 || n <= 0 || r <= 0) return 0;
  return big_layout(R, C, n, r).total;
}

int hla_big_impl(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows, int r, int bits,
                 int rounding, uint64_t seed, uint32_t rng_stream, int scale_mode, void* codes_out, int64_t ld_out,
                 float* scales_out, void* workspace, size_t workspace_bytes, hipStream_t st, const char* who,
                 hipEvent_t after_stats, float* row16_absmax_out, bool rowmajor, int store4) {
  const int m = n / 64;
  if (n < 256 || n > 8192 || (n & (n - 1))) return fail(HOT_ERR_UNSUPPORTED, "%s: block size %d (a power of two, 256 .. 8192)", who, n);
  const int64_t NB = R / n, kout = NB * r;
  if (!rowmajor && store4) return fail(HOT_ERR_UNSUPPORTED, "%s: blocks above 128 tokens have no transposed packed-INT4 store", who);
  if (store4 && (C & 1)) return fail(HOT_ERR_UNSUPPORTED, "%s: packed INT4 output needs an even number of channels", who);
  const int64_t row_bytes = rowmajor ? (store4 ? C / 2 : C) : kout;
  if (ld_out < row_bytes || (ld_out & 15)) return fail(HOT_ERR_INVALID, "%s: ld_out=%lld must be a multiple of 16 and >= %lld", who, (long long)ld_out, (long long)row_bytes);
  const BigLayout b = big_layout(R, C, n, r);
  if (!workspace || workspace_bytes < b.total) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, b.total, workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  const int64_t gx = (C + BT - 1) / BT;
  if (R / 64 > 65535 || (scale_mode == HOT_SCALE_SAWB && gx * NB * 64 > 65536))
    return fail(HOT_ERR_UNSUPPORTED, "%s: %lld blocks of %d tokens x %lld channels exceed the grid of the large-block path", who, (long long)NB, n, (long long)C);

  uint8_t* ws = (uint8_t*)workspace;
  BigArgs a;
  a.in = in; a.T = (float*)(ws + b.off_T); a.tmp = (int8_t*)(ws + b.off_tmp); a.tab = (const int32_t*)(ws + b.off_tab);
  a.R = R; a.C = C; a.NB = NB; a.n = n; a.r = r; a.rpad = r == 1 ? 1 : (r + 7) & ~7; a.bits = bits; a.rounding = rounding;
  a.mode = scale_mode; a.stat = (float*)ws; a.colmax = (float*)(ws + b.off_colmax);
  a.partial = (double*)(ws + b.off_partial); a.scales_out = scales_out; a.seed = seed; a.stream = rng_stream;
  a.tmp_ld = C;
  // the row table (and with it the check of the row list), after the clear kernel below
  uint64_t kmask = 0;
  for (int k = 0; k < r; ++k)
    if (rows[k] >= 0 && rows[k] < n) kmask |= 1ull << (rows[k] & 63);
  a.kmask = kmask; a.nk = 0;
  for (int k = 0; k < 64; ++k) {
    a.klist[k] = 0;
    if ((kmask >> k) & 1ull) a.klist[a.nk++] = (uint8_t)k;
  }
  if (NB * a.nk > 65535) return fail(HOT_ERR_UNSUPPORTED, "%s: %lld blocks of %d tokens exceed the grid of the large-block path", who, (long long)NB, n);

  // statistics and table cleared, then the table written piece by piece (rows in natural order, so
  // the visit number of a piece's entry i is its position in the sorted list)
  const int64_t nclr = std::max<int64_t>(std::max<int64_t>(C, n), (int64_t)(STAT_BYTES / 4));
  if (r <= TAB_ROWS) {
    // the row list is checked here, the table written by the clear launch itself
    std::unique_ptr<uint8_t[]> seen(new uint8_t[(size_t)n]());
    TabRows tr;
    memset(&tr, 0, sizeof(tr));
    tr.count = r;
    for (int k = 0; k < r; ++k) {
      if (rows[k] < 0 || rows[k] >= n) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d outside [0, %d)", who, k, rows[k], n);
      if (seen[(size_t)rows[k]]) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d listed twice", who, k, rows[k]);
      seen[(size_t)rows[k]] = 1;
      tab_row_put(tr.packed, k, rows[k]);
    }
    hipLaunchKernelGGL(big_prepare_kernel, dim3((unsigned)((nclr + 255) / 256)), dim3(256), 0, st, a.stat, a.colmax, C,
                       (int32_t*)(ws + b.off_tab), n, tr);
    if (int rc = check_launch("big_prepare_kernel")) return rc;
  } else {
    hipLaunchKernelGGL(big_clear_kernel, dim3((unsigned)((nclr + 255) / 256)), dim3(256), 0, st, a.stat, a.colmax, C,
                       (int32_t*)(ws + b.off_tab), n);
    if (int rc = build_row_table((int32_t*)(ws + b.off_tab), n, rows, r, nullptr, st, who)) return rc;
  }
  const dim3 g1((unsigned)gx, (unsigned)(R / 64));
  a.row_absmax = row16_absmax_out;
  if (row16_absmax_out && (C % 16 || scale_mode == HOT_SCALE_SAWB))
    return fail(HOT_ERR_UNSUPPORTED, "%s: fused row statistic unavailable for this configuration", who);
  switch (dtype) {
    case HOT_F32:
      if (row16_absmax_out) hipLaunchKernelGGL((big_stage1_kernel<float, true>), g1, dim3(BT), 0, st, a);
      else hipLaunchKernelGGL((big_stage1_kernel<float, false>), g1, dim3(BT), 0, st, a);
      break;
    case HOT_BF16:
      if (row16_absmax_out) hipLaunchKernelGGL((big_stage1_kernel<bf16_t, true>), g1, dim3(BT), 0, st, a);
      else hipLaunchKernelGGL((big_stage1_kernel<bf16_t, false>), g1, dim3(BT), 0, st, a);
      break;
    case HOT_F16:
      if (row16_absmax_out) hipLaunchKernelGGL((big_stage1_kernel<f16_t, true>), g1, dim3(BT), 0, st, a);
      else hipLaunchKernelGGL((big_stage1_kernel<f16_t, false>), g1, dim3(BT), 0, st, a);
      break;
    default: return fail(HOT_ERR_INVALID, "%s: bad dtype %d", who, dtype);
  }
  if (int rc = check_launch("big_stage1_kernel")) return rc;
  const dim3 g2((unsigned)gx, (unsigned)(NB * a.nk));
  if (int rc = dispatch_stage2(m, a, g2, 0, st)) return rc;
  // rows listed run-major (sorted by (row % 64, row / 64)): the quantise pass stores K-major itself
  bool run_major = !rowmajor && NB * ((a.nk + KG - 1) / KG) <= 65535;
  for (int k = 1; k < r && run_major; ++k) {
    const int prev = (rows[k - 1] & 63) * m + (rows[k - 1] >> 6), cur = (rows[k] & 63) * m + (rows[k] >> 6);
    run_major = cur > prev;
  }
  // (with absmax steps the run-major quantise pass reads the statistic itself and publishes the steps)
  if (!(run_major && scale_mode != HOT_SCALE_SAWB))
    hipLaunchKernelGGL(big_finalize_kernel, dim3(1), dim3(256), 0, st, a, (int64_t)gx * NB * a.nk, kout);
  if (after_stats) (void)hipEventRecord(after_stats, st);
  if (rowmajor) {
    // untransposed [NB r, C]: the quantise pass writes the destination itself (INT8), or its [Kout, C]
    // scratch, which a second kernel packs two channels to a byte
    if (!store4) { a.tmp = (int8_t*)codes_out; a.tmp_ld = ld_out; }
    if (int rc = dispatch_stage2(m, a, g2, 1, st)) return rc;
    if (store4) {
      const int64_t items = kout * (C / 2);
      hipLaunchKernelGGL(pack4_rows_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st, a.tmp, kout, C, (int8_t*)codes_out, ld_out);
      return check_launch("pack4_rows_kernel");
    }
    return HOT_OK;
  }
  if (run_major) {
    memset(a.keep, 0, sizeof(a.keep));
    memset(a.kbase, 0, sizeof(a.kbase));
    int kc = -1, last_k = -1;
    for (int i = 0; i < r; ++i) {
      const int k = rows[i] & 63, j = rows[i] >> 6;
      if (k != last_k) { ++kc; last_k = k; a.kbase[kc] = (uint16_t)i; }
      a.keep[kc][j >> 5] |= 1u << (j & 31);
    }
    for (int q = kc + 1; q <= 64; ++q) a.kbase[q] = (uint16_t)r;
    return dispatch_runs(m, a, codes_out, ld_out, st);
  }
  if (int rc = dispatch_stage2(m, a, g2, 1, st)) return rc;
  const dim3 gt((unsigned)((ld_out + 63) / 64), (unsigned)((C + 63) / 64));
  hipLaunchKernelGGL(transpose_i8_kernel, gt, dim3(256), 0, st, a.tmp, kout, C, (int8_t*)codes_out, ld_out);
  return check_launch("transpose_i8_kernel");
}

size_t hla_expand_big_workspace_bytes_impl(int64_t nb, int64_t C, int n) {
  return (size_t)round_up((int64_t)n * 4, 256) + (size_t)round_up(nb * n * C * 4, 256);
}

int hla_expand_big_impl(const float* t, int64_t nb, int64_t C, int n, const int32_t* rows, int r, float post, void* out,
                        int out_dtype, void* workspace, size_t workspace_bytes, hipStream_t st) {
  const char* who = "hla_expand";
  const int m = n / 64;
  if (n < 256 || n > 8192 || (n & (n - 1))) return fail(HOT_ERR_UNSUPPORTED, "%s: block size %d (a power of two, 256 .. 8192)", who, n);
  if (r < 1 || r > n) return fail(HOT_ERR_INVALID, "%s: r=%d outside [1, %d]", who, r, n);
  if (nb * m > 65535 || nb * 64 > 65535) return fail(HOT_ERR_UNSUPPORTED, "%s: %lld blocks of %d tokens exceed the grid", who, (long long)nb, n);
  const size_t need = hla_expand_big_workspace_bytes_impl(nb, C, n);
  if (!workspace || workspace_bytes < need) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  int32_t* tab = (int32_t*)workspace;
  ExpandBigArgs a;
  a.t = t; a.U = (float*)((uint8_t*)workspace + round_up((int64_t)n * 4, 256)); a.out = out; a.tab = tab; a.C = C;
  a.r = r; a.m = m; a.post = post;
  hipLaunchKernelGGL(tab_clear_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, tab, n);
  if (int rc = build_row_table(tab, n, rows, r, nullptr, st, who)) return rc;
  const unsigned gx = (unsigned)((C + BT - 1) / BT);
  hipLaunchKernelGGL(expand_runs_kernel, dim3(gx, (unsigned)(nb * m)), dim3(BT), 0, st, a);
  if (int rc = check_launch("expand_runs_kernel")) return rc;
  const dim3 g2(gx, (unsigned)(nb * 64));
  switch (m) {
    case 4: return launch_expand_across<4>(a, g2, out_dtype, st);
    case 8: return launch_expand_across<8>(a, g2, out_dtype, st);
    case 16: return launch_expand_across<16>(a, g2, out_dtype, st);
    case 32: return launch_expand_across<32>(a, g2, out_dtype, st);
    case 64: return launch_expand_across<64>(a, g2, out_dtype, st);
    default: return launch_expand_across<128>(a, g2, out_dtype, st);
  }
}

}  // namespace hot
