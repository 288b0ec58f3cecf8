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
// Data movement.  A workgroup owns 256 adjacent channels (columns) and a run
// of token blocks.  Rows arrive 16 at a time through coalesced 16-byte loads
// (each row of the tile is one contiguous segment of HBM), are parked in a
// double-buffered LDS tile, and every thread then pulls ITS channel's 16
// values out of LDS: from there on a thread holds whole columns, so the
// butterflies (stage order h = 1, 2, 4, ..., the canonical fp32 order) need
// no cross-lane traffic.  Quantised codes are staged in LDS as [channel][k]
// and leave the CU as one contiguous K-run per channel.  Two passes over the
// input (statistics, then quantise): the step of a tensor depends on all of it.
//
// HBM traffic per input element: 2 * sizeof(in) read + (r/n) * bits/8 written.
#include <mutex>

#include "hot_device.h"
#include "hot_host.h"

namespace hot {

constexpr int CW = 256;        // threads per workgroup = channels per workgroup
constexpr size_t COL_STAT_BYTES = 256 + STAT_SLOT_BYTES;   // step / clip words, then the absmax slots
constexpr int COLMAX_COPIES = 8;  // per-channel maxima: workgroup row y folds into copy y % 8 (fewer atomics per line)
constexpr int CW_ROWS = 16;    // rows staged per step

constexpr int GS = 32;   // floats between the statistics of two sample groups (one 128-byte line each)

struct ColArgs {
  const void* in;
  int64_t R, C;       // input rows (transform dim) and channels
  int64_t NB;         // token blocks = R / N
  int64_t Kout;       // NB * r codes per output row
  int8_t* out;
  int64_t ld_out;     // bytes
  float* stat;        // [1] step s, [2] clip (SAWB)
  float* slots;       // TENSOR: absmax in STAT_SLOTS partial maxima
  double* partial;    // SAWB: 2 doubles per workgroup
  float* colmax;      // ROW: per-channel absmax, COLMAX_COPIES arrays of C floats
  float* scales_out;
  float* row_absmax;  // statistics pass with RS != 0: absmax of the row-wise block Hadamard (STAT_SLOTS partial maxima)
  float* colsum;      // statistics pass: NULL or per-channel sums of the input, one row of C floats per run of token blocks
  uint64_t seed;
  uint32_t stream;
  int32_t r, rpad, bits, store4, rounding, mode, tb, stats_cleared;
  uint32_t gx, gy;     // logical grid: channel strips x runs of token blocks
  // Sample groups (3-D activations: one step per sample).  The R rows are `groups` samples of NBs
  // token blocks each; a workgroup's run of blocks never leaves its sample (`runs` runs per sample),
  // the codes of a sample take Kpad bytes of every output row (the tail zeroed), and the statistics
  // are kept per sample: gstat[GS g] (absmax, TENSOR), gstat[GS g + 1] / [GS g + 2] (step / clip,
  // SAWB) -- a 128-byte line per sample, since every workgroup of a sample updates its absmax
  // and updates of one line queue up behind each other at the memory side --, colmax[g * C + c] (ROW).  groups == 1: the whole input is one group with Kpad = ld_out.
  int32_t groups, runs;
  int64_t NBs, Kpad;
  float* gstat;
  // rowmajor: the codes are stored untransposed, [NB r, C] with ld_out bytes per coefficient row
  // (the A operand of a product whose K runs along the channels), instead of [C, NB r]
  int32_t rowmajor;
  hipEvent_t after_stats;  // host only: recorded between the statistics and the quantise pass
  int8_t slot[COL_MAX_N];  // output position of natural row i, -1 = dropped
};

// Which coefficients of a block are kept and where they go.  The generic policy reads the table
// from the kernel arguments; the presets make it a compile-time constant, which removes the
// per-coefficient scalar branches and lets the compiler drop the butterflies that only feed
// discarded coefficients.
struct SelRuntime { static constexpr bool STATIC = false; };
template <int N> struct SelFull {
  static constexpr bool STATIC = true;
  static constexpr int slot(int i) { return i; }
};
struct SelPy64 {  // make_WHT rule for n = 64: 36 coefficients, sequency order
  static constexpr bool STATIC = true;
  static constexpr int8_t TABLE[64] = {0,  35, 25, 26, 14, 33, 15, 32, 7,  -1, -1, -1, -1, -1, -1, -1, 3,  -1, 22, 29, 11, -1,
                                       18, -1, 4,  -1, 21, -1, 10, -1, 19, -1, 1,  -1, 24, 27, 13, 34, 16, 31, 6,  -1, -1, -1,
                                       8,  -1, -1, -1, 2,  -1, 23, 28, 12, -1, 17, 30, 5,  -1, -1, -1, 9,  -1, 20, -1};
  static constexpr int slot(int i) { return TABLE[i]; }
};
struct SelPy128 {  // make_WHT rule for n = 128: the n = 64 selection on the even rows, no odd row
  static constexpr bool STATIC = true;
  static constexpr int slot(int i) { return (i & 1) ? -1 : SelPy64::TABLE[i >> 1]; }
};
struct SelPaper16 {  // the 8 lowest sequencies of a 16-block
  static constexpr bool STATIC = true;
  static constexpr int8_t TABLE[16] = {0, -1, 7, -1, 3, -1, 4, -1, 1, -1, 6, -1, 2, -1, 5, -1};
  static constexpr int slot(int i) { return TABLE[i]; }
};

template <typename T> struct raw_of { typedef uint16_t type; };
template <> struct raw_of<float> { typedef uint32_t type; };

template <typename T> __device__ __forceinline__ float cvt_raw(typename raw_of<T>::type v);
template <> __device__ __forceinline__ float cvt_raw<float>(uint32_t v) { return as_f(v); }
template <> __device__ __forceinline__ float cvt_raw<bf16_t>(uint16_t v) { return as_f((uint32_t)v << 16); }
template <> __device__ __forceinline__ float cvt_raw<f16_t>(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }

// Unnormalised FWHT of the N-point groups of v[0..LEN), stages h = H0, 2 H0, 4 H0, ... (H0 = 2: the
// caller has run the first stage already)
template <int N, int LEN, int H0 = 1>
__device__ __forceinline__ void fwht_regs(float (&v)[LEN]) {
#pragma unroll
  for (int h = H0; h < N; h <<= 1) {
#pragma unroll
    for (int i = 0; i < LEN; ++i) {
      if ((i & h) == 0) {
        const float a = v[i], b = v[i + h];
        v[i] = a + b;
        v[i + h] = a - b;
      }
    }
  }
}

// Streams the rows of the workgroup's tile through a ring of LDS buffers with
// direct global -> LDS loads (16 bytes per lane, no registers in between).
// Step s covers rows [row0 + 16 s, +16); a buffer holds them as one
// [16 rows][64 channels] slice per wave.  A wave-wide load fills one contiguous
// KiB of the wave's own slice, i.e. 1024 / (64 sizeof(T)) rows.  Rows past the
// end of the input and channels past C are redirected to valid addresses: what
// they deliver is never consumed.
// LDS buffers in the ring (steps in flight behind the one in use = depth - 1): four for 16-bit
// inputs; 32-bit rows are twice as large, and three buffers keep a second workgroup on the CU.
template <typename T> constexpr int ring_depth() { return sizeof(T) == 4 ? 3 : 4; }

template <typename T>
struct RowStream {
  static constexpr int RB = 64 * (int)sizeof(T);                 // bytes per staged row of ONE wave (64 channels)
  static constexpr int WAVE_BYTES = CW_ROWS * RB;                // one wave's share of a step
  static constexpr int BUF_BYTES = (CW / 64) * WAVE_BYTES;       // all waves' shares of a step
  static constexpr int LPW = WAVE_BYTES / 1024;                  // DMA instructions per wave per step
  static constexpr int VPR = RB / 16;                            // 16-byte vectors per staged row
  static constexpr int RPC = 1024 / RB;                          // rows per KiB chunk (one DMA instruction)
  const uint8_t* base;   // &in[0][first channel of this wave] (or of the workgroup when the wave has none)
  uint32_t pitch;        // bytes per input row
  int64_t rows_total;
  int64_t row0;
  int nvec_row;          // valid 16-byte vectors per row for this wave (at least 1)
};

// s_waitcnt vmcnt(VM) lgkmcnt(0); vmcnt is split over bits 3:0 and 15:14
template <int VM>
__device__ __forceinline__ void wait_stream() {
  __builtin_amdgcn_s_waitcnt((VM & 0xF) | ((VM >> 4) << 14) | (0x7 << 4) | (0x0 << 8));
}

__device__ __forceinline__ void dma16_to_lds(uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
  // lds_addr and sbase are wave-uniform by construction; said explicitly, since the instruction takes
  // them in scalar registers and the compiler keeps a uniform value in a vector register when it was
  // computed past lane-dependent control flow.  (The builtin returns a signed int: every half goes
  // through uint32_t, or a low half with its top bit set would sign-extend over the high half.)
  const uint64_t b64 = (uint64_t)(uintptr_t)sbase;
  const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b64 >> 32));
  const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b64);
  const uint8_t* base = reinterpret_cast<const uint8_t*>(((uint64_t)b_hi << 32) | (uint64_t)b_lo);
  const uint32_t lds_u = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_u), "v"(voff), "s"(base)
               : "memory", "m0");
}

// Every wave streams the rows of its own 64 channels into its own slice of each ring buffer
// ([16 rows][64 channels]), so a wave waits for nothing but its own loads: no workgroup barrier
// in the streaming loop, and the four waves of a workgroup drift apart freely.
template <typename T>
__device__ __forceinline__ void rs_issue(const RowStream<T>& rs, uint32_t wave_lds, int step, int lane) {
  constexpr int VPR = RowStream<T>::VPR, RPC = RowStream<T>::RPC;
#pragma unroll
  for (int i = 0; i < RowStream<T>::LPW; ++i) {
    int64_t row = rs.row0 + (int64_t)step * CW_ROWS + i * RPC + lane / VPR;
    if (row >= rs.rows_total) row = rs.rows_total - 1;
    int vec = lane % VPR;
    if (vec >= rs.nvec_row) vec = rs.nvec_row - 1;
    dma16_to_lds(wave_lds + i * 1024, (uint32_t)row * rs.pitch + (uint32_t)vec * 16, rs.base);
  }
}

template <typename T>
__device__ __forceinline__ void rs_column(const uint8_t* wave_buf, int lane, float* v) {
  typedef typename raw_of<T>::type raw_t;
  const raw_t* p = reinterpret_cast<const raw_t*>(wave_buf) + lane;
#pragma unroll
  for (int i = 0; i < CW_ROWS; ++i) v[i] = cvt_raw<T>(p[i * 64]);
}

// ---- the kernel: PASS 0 = statistics, PASS 1 = quantise + transposed store ----

// RS (statistics pass only): when non-zero the pass also tracks the absmax of the ROW-wise block
// Hadamard (block RS along the channels) of the same input, so that the row-wise quantiser of g_y
// needs no statistics pass of its own.  Adjacent lanes hold adjacent channels, hence the row-wise
// butterflies run across lanes.
template <typename T, int N, int PASS, int ROUND, bool SAWB, typename SEL, int RS = 0>
__global__ void __launch_bounds__(CW) colwise_kernel(const ColArgs a) {
  constexpr int SPB = N >= CW_ROWS ? N / CW_ROWS : 1;        // steps per token block
  constexpr int BPS = N >= CW_ROWS ? 1 : CW_ROWS / N;        // token blocks per step
  constexpr int XL = N >= CW_ROWS ? N : CW_ROWS;             // values a thread holds
  constexpr int BUF = RowStream<T>::BUF_BYTES;
  extern __shared__ __align__(16) uint8_t lds[];
  __shared__ float s_max[CW / 64];
  __shared__ double s_sum[2][CW / 64];
  constexpr int CW_DEPTH = ring_depth<T>();
  uint8_t* const stage = lds + CW_DEPTH * BUF;               // PASS 1: codes [channel][k]

  // One-dimensional launch.  The hardware deals consecutive workgroups to the eight XCDs in turn;
  // each XCD takes a contiguous chunk of the logical order, which runs along the token blocks
  // of one channel strip: the workgroups an XCD runs side by side then write neighbouring runs
  // of the same output rows, and its L2 merges their partial lines.
  // (The statistics pass stores nothing and keeps the plain order, strips fastest.)
  const unsigned ngrid = a.gx * a.gy, chunk = (ngrid + 7u) >> 3;
  const unsigned wg_lin = PASS == 1 ? (blockIdx.x & 7u) * chunk + (blockIdx.x >> 3) : blockIdx.x;
  if (wg_lin >= ngrid) return;
  const unsigned bx = PASS == 1 ? wg_lin / a.gy : wg_lin % a.gx;
  const unsigned by = PASS == 1 ? wg_lin - bx * a.gy : wg_lin / a.gx;
  const unsigned wg_id = by * a.gx + bx;     // the numbering the ordered reductions use
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t cg0 = (int64_t)bx * CW;
  // Fused row statistic: within each group of 16 lanes the channels are dealt out so that the four
  // stages of the 16-point row transform pair lanes at the distances a single DPP operand reaches
  // (channel bit 0 <-> lane xor 1, bit 1 <-> xor 2, bit 2 <-> xor 15, bit 3 <-> xor 8).
  constexpr bool RSP = PASS == 0 && RS == 16;
  const int chan = RSP ? (tid ^ ((tid & 4) ? 0xB : 0)) : tid;   // channel of this thread within the workgroup
  const int64_t c = cg0 + chan;
  const bool active = c < a.C;
  const int sample = a.groups > 1 ? (int)(by / (unsigned)a.runs) : 0;
  const int run = (int)by - sample * a.runs;
  const int64_t blk_in = (int64_t)run * a.tb;                    // first block of the run within its sample
  const int64_t blk0 = (int64_t)sample * a.NBs + blk_in;
  int nblk = (int)((a.NBs - blk_in) < a.tb ? (a.NBs - blk_in) : a.tb);
  const int nsteps = (nblk * N + CW_ROWS - 1) / CW_ROWS;
  const int qmax = (1 << (a.bits - 1)) - 1;
  const int sb = a.tb * a.r;        // staged code bytes per channel
  const int pitch = sb + 4;

  RowStream<T> rs;
  rs.pitch = (uint32_t)(a.C * (int64_t)sizeof(T));
  rs.rows_total = a.R;
  rs.row0 = blk0 * N;
  {
    // channels of this wave that exist; a wave past the end streams the workgroup's first
    // channels instead (valid addresses, never consumed)
    int64_t cw0 = cg0 + 64 * wave;
    int64_t chans = a.C - cw0;
    if (chans <= 0) { cw0 = cg0; chans = a.C - cg0; }
    if (chans > 64) chans = 64;
    rs.base = reinterpret_cast<const uint8_t*>(a.in) + cw0 * (int64_t)sizeof(T);
    rs.nvec_row = (int)(chans * (int64_t)sizeof(T) / 16);
  }

  float d = 1.f, rcp = 1.f, clip = 0.f;
  if constexpr (PASS == 1) {
    // gaps of partial groups must read as 0; a workgroup with all its channels and blocks writes
    // every staged byte itself
    if (nblk < a.tb || cg0 + CW > a.C) {
      uint32_t* l32 = reinterpret_cast<uint32_t*>(stage);
      for (int i = tid; i < CW * pitch / 4; i += CW) l32[i] = 0u;
      __syncthreads();
    }
    // absmax modes read the statistic itself (no finalize kernel in between) and publish the step
    if (a.groups > 1) {
      if (a.mode == HOT_SCALE_ROW) {
        const float sc = (active ? a.colmax[(int64_t)sample * a.C + c] : 0.f) / (float)qmax;
        d = active ? sc + 1e-11f : 1.f;
        if (active && run == 0) a.scales_out[(int64_t)sample * a.C + c] = sc;
      } else if (a.mode == HOT_SCALE_TENSOR) {
        const float sc = a.gstat[GS * sample] / (float)qmax;
        d = sc + 1e-11f;
        if (bx == 0 && run == 0 && tid == 0) a.scales_out[sample] = sc;
      } else {
        d = a.gstat[GS * sample + 1] + 1e-11f;
        clip = a.gstat[GS * sample + 2];
      }
    } else if (a.mode == HOT_SCALE_ROW) {
      float cm = 0.f;
      if (active) {
#pragma unroll
        for (int k = 0; k < COLMAX_COPIES; ++k) cm = fmaxf(cm, a.colmax[k * a.C + c]);
      }
      const float sc = cm / (float)qmax;
      d = active ? sc + 1e-11f : 1.f;
      if (active && by == 0) a.scales_out[c] = sc;
    } else if (a.mode == HOT_SCALE_TENSOR) {
      const float sc = stat_slots_max(a.slots, lane) / (float)qmax;
      d = sc + 1e-11f;
      if (bx == 0 && by == 0 && tid == 0) a.scales_out[0] = sc;
    } else {
      d = a.stat[1] + 1e-11f;
      clip = a.stat[2];
    }
    rcp = 1.0f / d;
  }
  const float rcpk = rcp * 65536.0f;       // stochastic rounding works in units of 2^-16

  float cmax = 0.f, rmax = 0.f, csum = 0.f;
  double ssq = 0.0, sab = 0.0;
  float x[XL];

  // Transforms and consumes the token blocks held in x; `bl` is the group-local index of the first.
  philox_words u1 = {0u, 0u, 0u, 0u};
  auto consume = [&](int bl) {
    fwht_regs<N, XL, (RSP && N >= 2) ? 2 : 1>(x);   // the fused statistics pass runs stage h = 1 while loading
#pragma unroll
    for (int g = 0; g < BPS; ++g) {
      const int blk = bl + g;
      if (blk < nblk) {
        // coefficient 0 of a block is the sum of its tokens (row 0 of H is all ones)
        if constexpr (PASS == 0) csum += x[g * N];
        int visited = 0;      // kept coefficients of this block quantised so far (stochastic rounding)
        uint32_t u[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};   // 16-bit uniform integers of eight visits
        if constexpr (PASS == 1 && ROUND != HOT_ROUND_NEAREST && N == 1) {
          // blocks of one token keep their one coefficient: element number = channel * NB + block, so
          // eight consecutive blocks of a channel share a generator call (u1 lives across the blocks
          // of this step; a new call at the first block and wherever the number passes a multiple of 8)
          const uint64_t e = (uint64_t)c * (uint64_t)a.NB + (uint64_t)(blk0 + blk);
          if (g == 0 || (e & 7u) == 0) u1 = sr_octet_words(e >> 3, a.seed, a.stream);
          u[0] = sr_bits_of(u1, (uint32_t)e);
        }
#pragma unroll
        for (int i = 0; i < N; ++i) {
          int sl;
          if constexpr (SEL::STATIC) sl = SEL::slot(i); else sl = a.slot[i];
          if (sl >= 0) {
            float v = x[g * N + i];
            if constexpr (PASS == 0) {
              cmax = fmaxf(cmax, fabsf(v));
              if constexpr (SAWB) { ssq += (double)v * (double)v; sab += (double)fabsf(v); }
            } else {
              if constexpr (SAWB) v = fminf(fmaxf(v, -clip), clip);
              int q;
              if constexpr (ROUND == HOT_ROUND_NEAREST) {
                // |v / d| <= qmax (1 + 2^-22) by construction of d (absmax) or of the clip (SAWB):
                // the rounded code cannot leave [-qmax, qmax]
                q = (int)rint_div_fast(v, d, rcp);
              } else {
                // counter = ((channel * NB + block) * rpad + visit index) / 8, slot = visit index % 8
                // (blocks of one token: u[0] was drawn above)
                if (N > 1 && (visited & 7) == 0) {
                  if (a.r == 1) {
                    // a single kept coefficient per block: numbered channel * NB + block, like the
                    // one-token blocks above
                    const uint64_t e = (uint64_t)c * (uint64_t)a.NB + (uint64_t)(blk0 + blk);
                    u[0] = sr_bits_of(sr_octet_words(e >> 3, a.seed, a.stream), (uint32_t)e);
                  } else {
                    const uint64_t oct = ((uint64_t)c * (uint64_t)a.NB + (uint64_t)(blk0 + blk)) * (uint64_t)(a.rpad >> 3) +
                                         (uint64_t)(visited >> 3);
                    sr_bits8(oct, a.seed, a.stream, u);
                  }
                }
                q = q_stoch_fix(v, rcpk, u[visited & 7], qmax);   // (the minimum inside: floor + 1 may step past qmax at the very top)
                ++visited;
              }
              stage[tid * pitch + blk * a.r + sl] = (uint8_t)(q & 0xFF);
            }
          }
        }
      }
    }
  };

  // ring of CW_DEPTH LDS buffers: steps s+1 .. s+CW_DEPTH-1 are in flight while step s is consumed
  constexpr int LPW = RowStream<T>::LPW, WB = RowStream<T>::WAVE_BYTES;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t*)lds + wave * WB;
  const uint8_t* const my = lds + wave * WB;               // this wave's slice of ring buffer 0
#pragma unroll
  for (int s = 0; s < CW_DEPTH - 1; ++s)
    if (s < nsteps) rs_issue<T>(rs, lds0 + s * BUF, s, lane);
  // one step: wait for its rows, let the ring advance, pull this thread's 16 values into x[xo..]
  // -1 on the lane that holds the upper channel of a pair, per channel bit
  const float sg1 = (chan & 1) ? -1.f : 1.f, sg2 = (chan & 2) ? -1.f : 1.f;
  const float sg4 = (chan & 4) ? -1.f : 1.f, sg8 = (chan & 8) ? -1.f : 1.f;
  auto step = [&](int s, float* dst) {
    // this wave's rows of step s have landed, and its LDS reads of step s-1 are complete: the
    // slice that held step s-1 may be refilled.  Steps s+1 .. s+CW_DEPTH-2 may still be in flight.
    if (CW_DEPTH >= 4 && s + 2 < nsteps) wait_stream<2 * LPW>();
    else if (CW_DEPTH >= 3 && s + 1 < nsteps) wait_stream<LPW>();
    else wait_stream<0>();
    if (s + CW_DEPTH - 1 < nsteps) rs_issue<T>(rs, lds0 + ((s + CW_DEPTH - 1) % CW_DEPTH) * BUF, s + CW_DEPTH - 1, lane);
    if constexpr (RSP) {
      // Row-wise 16-point transform across lanes, magnitudes only.  A stage computes
      // own + s * partner with s = +1 on the lane of the lower channel of a pair (own + partner) and
      // -1 on the other (own - partner = -(partner - own)): a lane's value may come out negated,
      // but paired lanes agree in all lower channel bits and so carry the same sign, every value
      // stays +-(the true coefficient), and the product with +-1 is exact: the magnitudes are those
      // of the add/sub butterflies.  One v_fmac with a DPP operand per stage; the stages run
      // row-major over the 16 rows, so no DPP read follows the write of its register within two
      // instructions (and two wait states separate the rows' last writes from the first stage).
      // The raw rows are consumed here, so the first token-wise stage (rows 2j and 2j+1, always
      // within a step) is taken from them first.
      static_assert(CW_ROWS == 16, "the operand list below names sixteen rows");
      float t[CW_ROWS];
      rs_column<T>(my + (s % CW_DEPTH) * BUF, chan & 63, t);
      if constexpr (N >= 2) {
#pragma unroll
        for (int j = 0; j < CW_ROWS; j += 2) { dst[j] = t[j] + t[j + 1]; dst[j + 1] = t[j] - t[j + 1]; }
      } else {
#pragma unroll
        for (int j = 0; j < CW_ROWS; ++j) dst[j] = t[j];
      }
      // the first token-wise stage is complete before the rows are overwritten (else the compiler
      // keeps copies of them)
      asm volatile(""
                   : "+v"(dst[0]), "+v"(dst[1]), "+v"(dst[2]), "+v"(dst[3]), "+v"(dst[4]), "+v"(dst[5]), "+v"(dst[6]),
                     "+v"(dst[7]), "+v"(dst[8]), "+v"(dst[9]), "+v"(dst[10]), "+v"(dst[11]), "+v"(dst[12]),
                     "+v"(dst[13]), "+v"(dst[14]), "+v"(dst[15]));
      // every row is in its register before the first DPP read (the hazard check of the compiler
      // does not look into asm statements): the statement below takes all sixteen as operands
      asm volatile("s_nop 1"
                   : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]), "+v"(t[7]),
                     "+v"(t[8]), "+v"(t[9]), "+v"(t[10]), "+v"(t[11]), "+v"(t[12]), "+v"(t[13]), "+v"(t[14]), "+v"(t[15]));
#pragma unroll
      for (int i = 0; i < CW_ROWS; ++i)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "+v"(t[i]) : "v"(sg1));
#pragma unroll
      for (int i = 0; i < CW_ROWS; ++i)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "+v"(t[i]) : "v"(sg2));
#pragma unroll
      for (int i = 0; i < CW_ROWS; ++i)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 row_mirror row_mask:0xf bank_mask:0xf" : "+v"(t[i]) : "v"(sg4));
#pragma unroll
      for (int i = 0; i < CW_ROWS; ++i)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 row_ror:8 row_mask:0xf bank_mask:0xf" : "+v"(t[i]) : "v"(sg8));
#pragma unroll
      for (int i = 0; i < CW_ROWS; ++i) rmax = fmaxf(rmax, fabsf(t[i]));
      return;
    }
    rs_column<T>(my + (s % CW_DEPTH) * BUF, lane, dst);
    if constexpr (PASS == 0 && RS != 0) {
#pragma unroll
      for (int i = 0; i < CW_ROWS; ++i) {
        float t = dst[i];
        // lower lane: own + partner ; upper lane: partner - own == partner + (-own)
        t = as_f(as_u(t) ^ ((lane & 1) ? 0x80000000u : 0u)) + lane_xor<1>(t);
        t = as_f(as_u(t) ^ ((lane & 2) ? 0x80000000u : 0u)) + lane_xor<2>(t);
        t = as_f(as_u(t) ^ ((lane & 4) ? 0x80000000u : 0u)) + lane_xor<4>(t);
        t = as_f(as_u(t) ^ ((lane & 8) ? 0x80000000u : 0u)) + lane_xor<8>(t);
        if constexpr (RS >= 32) t = as_f(as_u(t) ^ ((lane & 16) ? 0x80000000u : 0u)) + lane_xor<16>(t);
        if constexpr (RS >= 64) t = as_f(as_u(t) ^ ((lane & 32) ? 0x80000000u : 0u)) + lane_xor<32>(t);
        rmax = fmaxf(rmax, fabsf(t));
      }
    }
  };
  if constexpr (N >= CW_ROWS) {
    for (int bl = 0; bl < nblk; ++bl) {
#pragma unroll
      for (int p = 0; p < SPB; ++p) step(bl * SPB + p, x + p * CW_ROWS);
      consume(bl);
    }
  } else {
    for (int s = 0; s < nsteps; ++s) {
      step(s, x);
      consume(s * BPS);
    }
  }

  if constexpr (PASS == 0) {
    if (a.colsum && active) a.colsum[(int64_t)by * a.C + c] = csum;
    if constexpr (RS != 0) {
      // rows past the end of the input were redirected to real rows and channels past C form whole
      // inactive blocks, so only the latter need masking
      float m = wave_max(active ? rmax : 0.f);
      if (lane == 0) s_max[wave] = m;
      __syncthreads();
      if (tid == 0) {
        float mm = s_max[0];
        for (int i = 1; i < CW / 64; ++i) mm = fmaxf(mm, s_max[i]);
        stat_slot_update(a.row_absmax, wg_id, mm);
      }
      __syncthreads();
    }
    if (a.mode == HOT_SCALE_ROW) {
      if (active) {
        if (a.groups > 1) atomic_max_nonneg(a.colmax + (int64_t)sample * a.C + c, cmax);
        else atomic_max_nonneg(a.colmax + (by % COLMAX_COPIES) * a.C + c, cmax);
      }
      return;
    }
    if (a.mode == HOT_SCALE_TENSOR) {
      float m = wave_max(active ? cmax : 0.f);
      if (lane == 0) s_max[wave] = m;
      __syncthreads();
      if (tid == 0) {
        float mm = s_max[0];
        for (int i = 1; i < CW / 64; ++i) mm = fmaxf(mm, s_max[i]);
        if (a.groups > 1) atomic_max_nonneg(a.gstat + GS * sample, mm);
        else stat_slot_update(a.slots, wg_id, mm);
      }
      return;
    }
    // SAWB: per-workgroup partial sums, reduced in a fixed order by the finalize kernel
    ssq = wave_sum(active ? ssq : 0.0);
    sab = wave_sum(active ? sab : 0.0);
    if (lane == 0) { s_sum[0][wave] = ssq; s_sum[1][wave] = sab; }
    __syncthreads();
    if (tid == 0) {
      double q = 0.0, b = 0.0;
      for (int i = 0; i < CW / 64; ++i) { q += s_sum[0][i]; b += s_sum[1][i]; }
      const int64_t wg = (int64_t)wg_id;
      a.partial[2 * wg] = q;
      a.partial[2 * wg + 1] = b;
    }
  } else {
    __syncthreads();
    if (a.rowmajor) {
      // untransposed store: coefficient row (blk0 + b) r + k takes one code of every channel; a
      // wave writes 64 adjacent bytes (INT8) or, two channels to a byte, 32 (packed INT4: the even
      // channel in bits 3:0)
      const int krun = nblk * a.r;
      int8_t* orow = a.out + blk0 * a.r * a.ld_out;
      for (int k = 0; k < krun; ++k, orow += a.ld_out) {
        const int code = stage[tid * pitch + k];
        if (a.store4) {
          const int hi = __shfl_xor(code, 1, 64);
          if (active && !(tid & 1)) orow[c >> 1] = (int8_t)((code & 0xF) | ((hi & 0xF) << 4));
        } else if (active) {
          orow[c] = (int8_t)code;
        }
      }
      return;
    }
    // flush: each channel's staged run is one contiguous global segment
    const bool last = blk_in + a.tb >= a.NBs;       // the run that ends its sample also zeroes the sample's tail
    const int out_sb = a.store4 ? sb / 2 : sb;
    const int64_t seg0 = (int64_t)sample * a.Kpad + (int64_t)run * out_sb;      // byte offset in the output row
    const int64_t seg_end = last ? (int64_t)(sample + 1) * a.Kpad : seg0 + out_sb;
    const int ndw = (int)((seg_end - seg0) / 4);            // output dwords per channel
    const int sdw = out_sb / 4;                             // of which staged
    const int nch = (int)((a.C - cg0) < CW ? (a.C - cg0) : CW);
    // output dword jd of a staged channel row (packing two codes per byte when store4)
    auto word = [&](const uint32_t* row, int jd) -> uint32_t {
      if (jd >= sdw) return 0u;
      if (a.store4) {
        const uint32_t lo = row[2 * jd], hi = row[2 * jd + 1];
        // bytes b0..b7 -> nibbles: byte j of the result = (b[2j+1] << 4) | (b[2j] & 15)
        const uint32_t l = (lo & 0x0F) | ((lo >> 4) & 0xF0) | ((lo >> 8) & 0x0F00) | ((lo >> 12) & 0xF000);
        const uint32_t h = (hi & 0x0F) | ((hi >> 4) & 0xF0) | ((hi >> 8) & 0x0F00) | ((hi >> 12) & 0xF000);
        return (l & 0xFFFF) | (h << 16);
      }
      return row[jd];
    };
    // consecutive threads walk along K within a channel, then on to the next channel; (ch, jd) of
    // position p = tid + k CW advance by a fixed step, so the loop carries them instead of dividing.
    // Units of 8 bytes when the segments allow it (half the store instructions), else of 4.
    const int unit = ((out_sb & 7) == 0 && (ndw & 1) == 0) ? 2 : 1;      // dwords per store
    const int nun = ndw / unit;                                          // units per channel
    const int total = nch * nun;
    const int step_ch = CW / nun, step_jd = CW - step_ch * nun;
    int ch = tid / nun, jd = tid - ch * nun;
    int8_t* dst = a.out + (cg0 + ch) * a.ld_out + seg0 + (int64_t)jd * 4 * unit;
    const int64_t step_dst = step_ch * a.ld_out + (int64_t)step_jd * 4 * unit, wrap_dst = a.ld_out - (int64_t)nun * 4 * unit;
    for (int p = tid; p < total; p += CW, ch += step_ch, jd += step_jd, dst += step_dst) {
      if (jd >= nun) { jd -= nun; ++ch; dst += wrap_dst; }
      const uint32_t* row = reinterpret_cast<const uint32_t*>(stage + ch * pitch);
      if (unit == 2) {
        uint2 w2;
        w2.x = word(row, 2 * jd);
        w2.y = word(row, 2 * jd + 1);
        *reinterpret_cast<uint2*>(dst) = w2;
      } else {
        *reinterpret_cast<uint32_t*>(dst) = word(row, jd);
      }
    }
  }
}

// ---- finalize: statistics -> step sizes ----------------------------------------

__global__ void __launch_bounds__(256) colwise_finalize_kernel(const ColArgs a, int64_t nwg) {
  __shared__ double s_q[256], s_b[256];
  const float qmax = (float)((1 << (a.bits - 1)) - 1);
  const int tid = threadIdx.x;
  if (a.mode == HOT_SCALE_ROW) {
    for (int64_t c = tid; c < a.C; c += 256) {
      float cm = 0.f;
      for (int k = 0; k < COLMAX_COPIES; ++k) cm = fmaxf(cm, a.colmax[k * a.C + c]);
      a.scales_out[c] = cm / qmax;
    }
    return;
  }
  if (a.mode == HOT_SCALE_TENSOR) {
    const float mx = stat_slots_max(a.slots, tid & 63);
    if (tid == 0) {
      const float s = mx / qmax;
      a.stat[1] = s;
      a.stat[2] = mx;
      a.scales_out[0] = s;
    }
    return;
  }
  // SAWB: one block per sample group adds up the partial sums of the group's workgroups (nwg each,
  // numbered run-major, so a group's workgroups are adjacent) in a fixed order
  const int64_t g = blockIdx.x;
  double q = 0.0, b = 0.0;
  for (int64_t i = tid; i < nwg; i += 256) { q += a.partial[2 * (g * nwg + i)]; b += a.partial[2 * (g * nwg + i) + 1]; }
  s_q[tid] = q; s_b[tid] = b;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) { s_q[tid] += s_q[tid + s]; s_b[tid] += s_b[tid + s]; }
    __syncthreads();
  }
  if (tid == 0) {
    const double cnt = (double)(a.Kout / a.groups) * (double)a.C;
    const float clip = (float)(12.1 * sqrt(s_q[0] / cnt) - 12.2 * (s_b[0] / cnt));
    const float s = clip / qmax;
    if (a.groups > 1) {
      a.gstat[GS * g + 1] = s;
      a.gstat[GS * g + 2] = clip;
      a.scales_out[g] = s;
    } else {
      a.stat[1] = s;
      a.stat[2] = clip;
      a.scales_out[0] = s;
    }
  }
}

// stat | slots are adjacent (COL_STAT_BYTES); row_absmax is another slot array
__global__ void colwise_clear_kernel(float* stat, float* colmax, int64_t ncolmax, float* row_absmax, float* gstat, int64_t ngstat) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < (int64_t)(COL_STAT_BYTES / 4)) stat[i] = 0.f;
  if (row_absmax && i < (int64_t)(STAT_SLOT_BYTES / 4)) row_absmax[i] = 0.f;
  if (colmax && i < ncolmax) colmax[i] = 0.f;
  if (gstat && i < ngstat) gstat[i] = 0.f;
}

// ---- column sums ------------------------------------------------------------------

// Sums of a strip of rows per channel, thread = channel: the stand-alone form of what the statistics
// pass of colwise_kernel delivers for free (used when the token blocks take the two-level path).
template <typename T>
__global__ void __launch_bounds__(256) colsum_strip_kernel(const void* in, int64_t R, int64_t C, int64_t rows_per_wg,
                                                            float* partial) {
  typedef typename raw_of<T>::type raw_t;
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_wg;
  const int64_t r1 = r0 + rows_per_wg < R ? r0 + rows_per_wg : R;
  const raw_t* p = reinterpret_cast<const raw_t*>(in) + r0 * C + c;
  float acc = 0.f;
  int64_t r = r0;
  for (; r + 8 <= r1; r += 8, p += 8 * C) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = cvt_raw<T>(p[i * C]);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc += v[i];
  }
  for (; r < r1; ++r, p += C) acc += cvt_raw<T>(*p);
  partial[(int64_t)blockIdx.y * C + c] = acc;
}

// out[c] = sum of partial[s][c] over the strips s, rounded once to the output type, in a fixed order:
// eight groups of threads take the strips s = g, g + 8, g + 16, ... of a channel (eight loads in
// flight each, added in strip order), then the eight group sums are added in group order.  A
// workgroup covers 32 channels, so that a few hundred strips are a short chain of loads per thread.
constexpr int CS_GROUPS = 8, CS_CHANS = 32;
template <typename OutT>
__global__ void __launch_bounds__(CS_GROUPS * CS_CHANS) colsum_finish_kernel(const float* partial, int strips, int64_t C, OutT* out) {
  __shared__ float s_part[CS_GROUPS][CS_CHANS];
  const int ch = threadIdx.x % CS_CHANS, g = threadIdx.x / CS_CHANS;
  const int64_t c = (int64_t)blockIdx.x * CS_CHANS + ch;
  float acc = 0.f;
  if (c < C) {
    int s = g;
    for (; s + 7 * CS_GROUPS < strips; s += 8 * CS_GROUPS) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = partial[(int64_t)(s + i * CS_GROUPS) * C + c];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc += v[i];
    }
    for (; s < strips; s += CS_GROUPS) acc += partial[(int64_t)s * C + c];
  }
  s_part[g][ch] = acc;
  __syncthreads();
  if (g == 0 && c < C) {
    float t = s_part[0][ch];
#pragma unroll
    for (int i = 1; i < CS_GROUPS; ++i) t += s_part[i][ch];
    store_scalar<OutT>(out + c, t);
  }
}

// ---- host ---------------------------------------------------------------------


size_t colwise_stats_bytes_impl(int64_t C) { return COL_STAT_BYTES + (size_t)round_up(C * 4 * COLMAX_COPIES, 256); }

size_t hla_workspace_bytes_impl(int64_t R, int64_t C, int n, int r) {
  return n > COL_MAX_N ? hla_big_workspace_bytes_impl(R, C, n, r) : colwise_workspace_bytes_impl(C);
}

size_t colwise_workspace_bytes_impl(int64_t C) {
  // stat | per-channel max | per-workgroup partial sums (at most 65536 workgroups)
  return COL_STAT_BYTES + (size_t)round_up(C * 4 * COLMAX_COPIES, 256) + (size_t)(2 * sizeof(double)) * 65536;
}

// with sample groups: stat | per-sample per-channel max | per-sample statistics | partial sums
static size_t group_colmax_bytes(int64_t C, int groups) { return (size_t)round_up(C * 4 * (int64_t)groups, 256); }
static size_t group_gstat_bytes(int groups) { return (size_t)round_up((int64_t)groups * GS * 4, 256); }
size_t colwise_group_workspace_bytes_impl(int64_t C, int groups) {
  if (groups <= 1) return colwise_workspace_bytes_impl(C);
  return COL_STAT_BYTES + group_colmax_bytes(C, groups) + group_gstat_bytes(groups) + (size_t)(2 * sizeof(double)) * 65536;
}

template <typename T, int N, int PASS, int ROUND, bool SAWB, typename SEL, int RS = 0>
static int launch_pass(const ColArgs& a, dim3 grid, size_t lds, hipStream_t st) {
  // one-time per instantiation; later calls only read the outcome
  static std::once_flag attr_once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(attr_once, [] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&colwise_kernel<T, N, PASS, ROUND, SAWB, SEL, RS>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
  });
  if (attr_err != hipSuccess) return check_hip(attr_err, "hipFuncSetAttribute(colwise_kernel)");
  ColArgs b = a;
  b.gx = grid.x; b.gy = grid.y;
  const unsigned total = grid.x * grid.y;
  hipLaunchKernelGGL((colwise_kernel<T, N, PASS, ROUND, SAWB, SEL, RS>), dim3(((total + 7u) >> 3) << 3), dim3(CW), lds, st, b);
  return HOT_OK;
}

// Token blocks per workgroup of the quantise pass (tb) and of an absmax statistics pass (tb0).
// The staged run of a channel (tb * r codes) must be a whole number of output dwords and cover the
// blocks that share a 16-row step, and is at least 32 bytes long.  Beyond that, runs grow (up to 128
// bytes) only while the grid keeps four workgroups per CU and the staging area does not cost a
// resident workgroup: with the ring of a 16-bit input three workgroups share a CU up to 80 staged
// bytes per channel, and the quantise pass lost a quarter of its speed each time a longer run took
// one away (measured at 8192 x 11008 and 11008 x 4096; the L2 of an XCD merges the short runs of
// neighbouring workgroups anyway).  (Runs below 32 bytes make a small W kernel faster on its own,
// 8 us instead of 11 at 3072 x 768, but its four times as many workgroups then get in the way of the
// g_y statistics pass it runs beside: the step came out 2 us slower.)  Absmax statistics stage nothing: while the grid has fewer than 2048
// workgroups they take shorter workgroups, down to 64 rows (measured 1 us faster at 12608 x 3072).
// The SAWB sums are order-sensitive and keep the partition of the quantise pass.
struct ColPartition { int tb, tb0; };
static ColPartition col_partition(int n, int r, int store4, int mode, int64_t C, int64_t NB, int elem_bytes) {
  const int BPS = n >= CW_ROWS ? 1 : CW_ROWS / n;
  const int64_t gx = (C + CW - 1) / CW;
  const size_t ring = (size_t)(elem_bytes == 4 ? 3 : 4) * CW_ROWS * CW * elem_bytes;
  auto run_bytes = [&](int t) { return store4 ? t * r / 2 : t * r; };   // t * r is a multiple of 8 when store4
  auto wgs = [&](int t) { return gx * ((NB + t - 1) / t); };
  auto resident = [&](int t) {   // workgroups of the quantise pass per CU, as far as LDS decides (three are enough)
    const size_t per = ring + (size_t)CW * (t * r + 4) + 256;
    const int k = (int)((160u * 1024u) / per);
    return k > 3 ? 3 : k;
  };
  int tb = BPS;
  while ((tb * r) % (store4 ? 8 : 4) != 0 || run_bytes(tb) < 32) tb <<= 1;
  while (run_bytes(tb) < 128 && wgs(2 * tb) >= 1024 && resident(2 * tb) >= resident(tb)) tb <<= 1;
  int tb0 = tb;
  if (mode != HOT_SCALE_SAWB)
    while (tb0 > BPS && (tb0 & 1) == 0 && tb0 * n > 64 && wgs(tb0) < 2048) tb0 >>= 1;
  return {tb, tb0};
}

template <typename T, int N, typename SEL>
static int launch_colwise(ColArgs& a, hipStream_t st) {
  const ColPartition part = col_partition(N, a.r, a.store4, a.mode, a.C, a.NB, (int)sizeof(T));
  const int tb = part.tb;
  a.tb = tb;
  const size_t in_bytes = (size_t)ring_depth<T>() * CW_ROWS * CW * sizeof(T);
  const size_t lds_stats = in_bytes, lds_quant = in_bytes + (size_t)CW * (tb * a.r + 4);
  if (lds_quant > 150 * 1024) return fail(HOT_ERR_UNSUPPORTED, "colwise: staging does not fit LDS");
  // runs of token blocks: per sample group (a run never leaves its sample)
  const int64_t gx = (a.C + CW - 1) / CW, runs = (a.NBs + tb - 1) / tb, gy = runs * a.groups;
  if (gy > 65535 || gx * gy > 65536) return fail(HOT_ERR_UNSUPPORTED, "colwise: grid %lld x %lld too large", (long long)gx, (long long)gy);
  a.runs = (int)runs;
  const dim3 grid((unsigned)gx, (unsigned)gy);
  if (!a.stats_cleared) {
    const int64_t ncolmax = a.mode == HOT_SCALE_ROW ? (a.groups > 1 ? a.C * a.groups : a.C * COLMAX_COPIES) : 0;
    const int64_t ngstat = a.groups > 1 ? GS * (int64_t)a.groups : 0;
    int64_t nclr = (int64_t)(COL_STAT_BYTES / 4);
    if (ncolmax > nclr) nclr = ncolmax;
    if (ngstat > nclr) nclr = ngstat;
    hipLaunchKernelGGL(colwise_clear_kernel, dim3((unsigned)((nclr + 255) / 256)), dim3(256), 0, st, a.stat,
                       ncolmax ? a.colmax : (float*)nullptr, ncolmax, a.row_absmax, ngstat ? a.gstat : (float*)nullptr, ngstat);
  }
  int rc;
  if (a.mode == HOT_SCALE_SAWB) {
    rc = launch_pass<T, N, 0, 0, true, SEL>(a, grid, lds_stats, st);   // same partition as ever: the sums are order-sensitive
  } else {
    ColArgs a0 = a;
    a0.tb = part.tb0;
    a0.runs = (int)((a.NBs + a0.tb - 1) / a0.tb);
    const dim3 grid0((unsigned)gx, (unsigned)(a0.runs * a.groups));
    if (a.row_absmax) rc = launch_pass<T, N, 0, 0, false, SEL, 16>(a0, grid0, lds_stats, st);
    else rc = launch_pass<T, N, 0, 0, false, SEL>(a0, grid0, lds_stats, st);
  }
  if (rc) return rc;
  if (a.mode == HOT_SCALE_SAWB) hipLaunchKernelGGL(colwise_finalize_kernel, dim3((unsigned)a.groups), dim3(256), 0, st, a, gx * runs);
  if (a.after_stats) (void)hipEventRecord(a.after_stats, st);
  if (a.rounding == HOT_ROUND_STOCH) {
    if (a.mode == HOT_SCALE_SAWB) rc = launch_pass<T, N, 1, 1, true, SEL>(a, grid, lds_quant, st);
    else rc = launch_pass<T, N, 1, 1, false, SEL>(a, grid, lds_quant, st);
  } else {
    if (a.mode == HOT_SCALE_SAWB) rc = launch_pass<T, N, 1, 0, true, SEL>(a, grid, lds_quant, st);
    else rc = launch_pass<T, N, 1, 0, false, SEL>(a, grid, lds_quant, st);
  }
  if (rc) return rc;
  return check_launch("colwise_kernel");
}

// Rows of the partial column sums a token-wise call writes: one per run of token blocks of its
// statistics pass; the stand-alone kernel of the large-block path takes strips of at least 64 rows,
// about 2048 workgroups in all.
static int64_t colsum_strip_rows_big(int64_t R, int64_t C) {
  const int64_t gx = (C + 255) / 256;
  const int64_t want = 2048 / gx > 0 ? 2048 / gx : 1;
  const int64_t rows = round_up((R + want - 1) / want, 16);
  return rows < 64 ? 64 : rows;
}

int64_t colsum_strips_impl(int64_t R, int64_t C, int n, int r, int store4, int mode, int elem_bytes) {
  if (R <= 0 || C <= 0 || n < 1 || r < 1) return 0;
  if (n > COL_MAX_N) {
    const int64_t rows = colsum_strip_rows_big(R, C);
    return (R + rows - 1) / rows;
  }
  const int64_t NB = R / n;
  const ColPartition part = col_partition(n, r, store4, mode, C, NB, elem_bytes);
  return (NB + part.tb0 - 1) / part.tb0;
}

int colsum_finish_impl(const float* partial, int64_t strips, int64_t C, void* out, int out_dtype, hipStream_t st) {
  const dim3 grid((unsigned)((C + CS_CHANS - 1) / CS_CHANS)), block(CS_GROUPS * CS_CHANS);
  switch (out_dtype) {
    case HOT_F32: hipLaunchKernelGGL(colsum_finish_kernel<float>, grid, block, 0, st, partial, (int)strips, C, (float*)out); break;
    case HOT_BF16: hipLaunchKernelGGL(colsum_finish_kernel<bf16_t>, grid, block, 0, st, partial, (int)strips, C, (bf16_t*)out); break;
    case HOT_F16: hipLaunchKernelGGL(colsum_finish_kernel<f16_t>, grid, block, 0, st, partial, (int)strips, C, (f16_t*)out); break;
    default: return fail(HOT_ERR_INVALID, "column sums: bad output dtype %d", out_dtype);
  }
  return check_launch("colsum_finish_kernel");
}

template <typename SEL, int N>
static bool matches(const ColArgs& a) {
  for (int i = 0; i < N; ++i)
    if (a.slot[i] != SEL::slot(i)) return false;
  return true;
}

template <typename T>
static int dispatch_colwise_n(int n, ColArgs& a, hipStream_t st) {
  switch (n) {
    case 1: return launch_colwise<T, 1, SelFull<1>>(a, st);   // r = 1 is the only choice
    case 2: return launch_colwise<T, 2, SelRuntime>(a, st);
    case 4: return launch_colwise<T, 4, SelRuntime>(a, st);
    case 8: return launch_colwise<T, 8, SelRuntime>(a, st);
    case 16:
      if (a.r == 16 && matches<SelFull<16>, 16>(a)) return launch_colwise<T, 16, SelFull<16>>(a, st);
      if (a.r == 8 && matches<SelPaper16, 16>(a)) return launch_colwise<T, 16, SelPaper16>(a, st);
      return launch_colwise<T, 16, SelRuntime>(a, st);
    case 32:
      if (a.r == 32 && matches<SelFull<32>, 32>(a)) return launch_colwise<T, 32, SelFull<32>>(a, st);
      return launch_colwise<T, 32, SelRuntime>(a, st);
    case 64:
      if (a.r == 36 && matches<SelPy64, 64>(a)) return launch_colwise<T, 64, SelPy64>(a, st);
      if (a.r == 64 && matches<SelFull<64>, 64>(a)) return launch_colwise<T, 64, SelFull<64>>(a, st);
      return launch_colwise<T, 64, SelRuntime>(a, st);
    case 128:
      if (a.r == 36 && matches<SelPy128, 128>(a)) return launch_colwise<T, 128, SelPy128>(a, st);
      return launch_colwise<T, 128, SelRuntime>(a, st);
    default: return fail(HOT_ERR_UNSUPPORTED, "colwise: block size %d (power of two up to %d)", n, COL_MAX_N);
  }
}

int colwise_quant_impl(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows, int r,
                       int bits, int rounding, uint64_t seed, uint32_t rng_stream, int scale_mode,
                       void* codes_out, int64_t ld_out, int store4, float* scales_out, void* workspace,
                       size_t workspace_bytes, hipStream_t st, const char* who, float* row16_absmax_out,
                       bool stats_cleared, hipEvent_t after_stats, float* colsum_partial, int groups, int64_t kpad_group,
                       bool rowmajor) {
  if (!in || !codes_out || !scales_out || !rows) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (rowmajor && (groups > 1 || scale_mode == HOT_SCALE_ROW || row16_absmax_out || colsum_partial))
    return fail(HOT_ERR_UNSUPPORTED, "%s: the untransposed store takes one step for the tensor and no fused statistics", who);
  if (R <= 0 || C <= 0) return fail(HOT_ERR_INVALID, "%s: bad shape R=%lld C=%lld", who, (long long)R, (long long)C);
  if (groups < 1) return fail(HOT_ERR_INVALID, "%s: %d sample groups", who, groups);
  if (groups > 1) {
    if (n > COL_MAX_N || store4 || row16_absmax_out || colsum_partial || stats_cleared)
      return fail(HOT_ERR_UNSUPPORTED, "%s: per-sample steps take token blocks up to %d, INT8 storage, and neither the fused row statistic nor the column sums", who, COL_MAX_N);
    if (n < 1 || R % ((int64_t)n * groups)) return fail(HOT_ERR_INVALID, "%s: R=%lld is not %d samples of whole blocks of %d", who, (long long)R, groups, n);
    if (kpad_group < (R / n / groups) * r || (kpad_group & 15)) return fail(HOT_ERR_INVALID, "%s: %lld code bytes per sample must be a multiple of 16 and hold the sample's codes", who, (long long)kpad_group);
  }
  if (n > COL_MAX_N) {
    // blocks one thread cannot hold: the two-level path
    if (store4 && !rowmajor) return fail(HOT_ERR_UNSUPPORTED, "%s: blocks above %d tokens have no transposed packed-INT4 store", who, COL_MAX_N);
    if (R % n) return fail(HOT_ERR_INVALID, "%s: R=%lld is not a multiple of the block %d", who, (long long)R, n);
    if (r < 1 || r > n) return fail(HOT_ERR_INVALID, "%s: r=%d outside [1, %d]", who, r, n);
    if (bits != 4 && bits != 8) return fail(HOT_ERR_UNSUPPORTED, "%s: bits=%d (4 or 8)", who, bits);
    if (rounding != HOT_ROUND_NEAREST && rounding != HOT_ROUND_STOCH) return fail(HOT_ERR_INVALID, "%s: bad rounding %d", who, rounding);
    if (scale_mode < HOT_SCALE_TENSOR || scale_mode > HOT_SCALE_SAWB) return fail(HOT_ERR_INVALID, "%s: bad scale mode %d", who, scale_mode);
    if (colsum_partial) {
      const int64_t rows = colsum_strip_rows_big(R, C);
      const dim3 grid((unsigned)((C + 255) / 256), (unsigned)((R + rows - 1) / rows));
      switch (dtype) {
        case HOT_F32: hipLaunchKernelGGL(colsum_strip_kernel<float>, grid, dim3(256), 0, st, in, R, C, rows, colsum_partial); break;
        case HOT_BF16: hipLaunchKernelGGL(colsum_strip_kernel<bf16_t>, grid, dim3(256), 0, st, in, R, C, rows, colsum_partial); break;
        case HOT_F16: hipLaunchKernelGGL(colsum_strip_kernel<f16_t>, grid, dim3(256), 0, st, in, R, C, rows, colsum_partial); break;
        default: return fail(HOT_ERR_INVALID, "%s: bad dtype %d", who, dtype);
      }
    }
    return hla_big_impl(in, dtype, R, C, n, rows, r, bits, rounding, seed, rng_stream, scale_mode, codes_out, ld_out,
                        scales_out, workspace, workspace_bytes, st, who, after_stats, row16_absmax_out, rowmajor, store4);
  }
  if (n < 1 || (n & (n - 1))) return fail(HOT_ERR_UNSUPPORTED, "%s: block size %d (a power of two)", who, n);
  if (R % n) return fail(HOT_ERR_INVALID, "%s: R=%lld is not a multiple of the block %d", who, (long long)R, n);
  if (r < 1 || r > n) return fail(HOT_ERR_INVALID, "%s: r=%d outside [1, %d]", who, r, n);
  if (bits != 4 && bits != 8) return fail(HOT_ERR_UNSUPPORTED, "%s: bits=%d (4 or 8)", who, bits);
  if (rounding != HOT_ROUND_NEAREST && rounding != HOT_ROUND_STOCH) return fail(HOT_ERR_INVALID, "%s: bad rounding %d", who, rounding);
  if (scale_mode < HOT_SCALE_TENSOR || scale_mode > HOT_SCALE_SAWB) return fail(HOT_ERR_INVALID, "%s: bad scale mode %d", who, scale_mode);
  if (C % 8) return fail(HOT_ERR_UNSUPPORTED, "%s: channel count %lld must be a multiple of 8", who, (long long)C);
  if (((uintptr_t)in & 15) || ((uintptr_t)codes_out & 15)) return fail(HOT_ERR_INVALID, "%s: pointers must be 16-byte aligned", who);
  if (R * C * 4 >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "%s: input of %lld x %lld elements exceeds the 32-bit offsets of the loader", who, (long long)R, (long long)C);

  ColArgs a;
  a.in = in; a.R = R; a.C = C; a.NB = R / n; a.Kout = a.NB * r;
  a.out = (int8_t*)codes_out; a.ld_out = ld_out;
  a.seed = seed; a.stream = rng_stream;
  a.r = r; a.rpad = (r + 7) & ~7; a.bits = bits; a.rounding = rounding; a.mode = scale_mode; a.tb = 4;
  for (int i = 0; i < COL_MAX_N; ++i) a.slot[i] = -1;
  for (int k = 0; k < r; ++k) {
    if (rows[k] < 0 || rows[k] >= n) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d outside [0, %d)", who, k, rows[k], n);
    if (a.slot[rows[k]] != -1) return fail(HOT_ERR_INVALID, "%s: rows[%d]=%d listed twice", who, k, rows[k]);
    a.slot[rows[k]] = (int8_t)k;
  }
  const int64_t row_bytes = rowmajor ? (store4 ? C / 2 : C) : groups > 1 ? kpad_group * groups : (store4 ? a.Kout / 2 : a.Kout);
  // packed INT4 pairs codes along K: a channel's codes must come in whole bytes (pairs along the channels
  // when the store is untransposed: C is a multiple of 8)
  if (store4 && !rowmajor && (a.Kout & 1)) return fail(HOT_ERR_UNSUPPORTED, "%s: packed INT4 output needs an even number of codes per channel", who);
  if (ld_out < row_bytes || (ld_out & 15)) return fail(HOT_ERR_INVALID, "%s: ld_out=%lld must be a multiple of 16 and >= %lld", who, (long long)ld_out, (long long)row_bytes);
  if (!workspace || workspace_bytes < colwise_group_workspace_bytes_impl(C, groups)) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed", who, colwise_group_workspace_bytes_impl(C, groups));
  if ((uintptr_t)workspace & 255) return fail(HOT_ERR_INVALID, "%s: workspace must be 256-byte aligned", who);
  a.store4 = store4;
  a.stats_cleared = stats_cleared ? 1 : 0;
  a.after_stats = after_stats;
  uint8_t* ws = (uint8_t*)workspace;
  a.stat = (float*)ws;
  a.slots = (float*)(ws + 256);
  a.colmax = (float*)(ws + COL_STAT_BYTES);
  a.partial = (double*)(ws + COL_STAT_BYTES + round_up(C * 4 * COLMAX_COPIES, 256));
  a.gstat = nullptr;
  a.rowmajor = rowmajor ? 1 : 0;
  a.groups = groups; a.runs = 1; a.NBs = a.NB / groups; a.Kpad = groups > 1 ? kpad_group : ld_out;
  if (groups > 1) {
    a.gstat = (float*)(ws + COL_STAT_BYTES + group_colmax_bytes(C, groups));
    a.partial = (double*)(ws + COL_STAT_BYTES + group_colmax_bytes(C, groups) + group_gstat_bytes(groups));
  }
  a.scales_out = scales_out;
  // the fused row-wise statistic exists for block 16 and absmax steps, and needs whole 16-blocks of channels
  a.colsum = colsum_partial;
  a.row_absmax = (row16_absmax_out && scale_mode != HOT_SCALE_SAWB && C % 16 == 0) ? row16_absmax_out : nullptr;
  if (row16_absmax_out && !a.row_absmax) return fail(HOT_ERR_UNSUPPORTED, "%s: fused row statistic unavailable for this configuration", who);
  switch (dtype) {
    case HOT_F32: return dispatch_colwise_n<float>(n, a, st);
    case HOT_BF16: return dispatch_colwise_n<bf16_t>(n, a, st);
    case HOT_F16: return dispatch_colwise_n<f16_t>(n, a, st);
    default: return fail(HOT_ERR_INVALID, "%s: bad dtype %d", who, dtype);
  }
}

// ---- the entry point that allocates nothing ---------------------------------------
//
// hot_hla_tokenwise needs a workspace (statistics words, per-channel maxima, per-workgroup sums).
// For callers that cannot allocate one, the same kernels run on a fixed array in device memory
// that is part of the library's code object: every GPU that loads the library holds one copy of
// it until the process ends.  Its size fixes the largest channel count the entry point takes.
constexpr int64_t STATIC_MAX_C = HOT_STATIC_MAX_CHANNELS;
constexpr size_t STATIC_SCRATCH_BYTES =
    COL_STAT_BYTES + (size_t)STATIC_MAX_C * 4 * COLMAX_COPIES + (size_t)(2 * sizeof(double)) * 65536;
static_assert((STATIC_MAX_C * 4 * COLMAX_COPIES) % 256 == 0, "the per-channel maxima end on a 256-byte boundary");
static __device__ __align__(256) uint8_t scratch[STATIC_SCRATCH_BYTES];

// Device address of `scratch` on the current device.  In host code the array's name is only a
// handle for the runtime, never an address a kernel could use; the address is asked for once per
// device (with that device current) and kept.
static int static_scratch_ptr(uint8_t** out, const char* who) {
  static std::mutex mu;
  static uint8_t* ptr[64] = {};
  int dev = -1;
  if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
  if (dev < 0 || dev >= 64) return fail(HOT_ERR_UNSUPPORTED, "%s: device index %d outside [0, 64)", who, dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void* p = nullptr;
    if (int rc = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
    if (!p || ((uintptr_t)p & 255)) return fail(HOT_ERR_HIP, "%s: the scratch array has no usable device address", who);
    ptr[dev] = (uint8_t*)p;
  }
  *out = ptr[dev];
  return HOT_OK;
}

}  // namespace hot

extern "C" int hot_hla_tokenwise_static(const void* in, int dtype, int64_t R, int64_t C, int n, const int32_t* rows,
                                        int r, int bits, int rounding, uint64_t seed, uint32_t rng_stream,
                                        int scale_mode, void* codes_out, int64_t ld_out, float* scales_out,
                                        void* hip_stream) {
  using namespace hot;
  const char* who = "hot_hla_tokenwise_static";
  if (n > COL_MAX_N)
    return fail(HOT_ERR_UNSUPPORTED, "%s: token blocks above %d need a workspace as large as the input; use hot_hla_tokenwise", who, COL_MAX_N);
  if (C > STATIC_MAX_C)
    return fail(HOT_ERR_UNSUPPORTED, "%s: %lld channels exceed the %lld the built-in scratch array holds; use hot_hla_tokenwise", who,
                (long long)C, (long long)STATIC_MAX_C);
  uint8_t* ws = nullptr;
  if (int rc = static_scratch_ptr(&ws, who)) return rc;
  // the statistics words at the head of the array are cleared by the first kernel of the call
  // (stats_cleared = false), everything else is written before it is read
  return colwise_quant_impl(in, dtype, R, C, n, rows, r, bits, rounding, seed, rng_stream, scale_mode, codes_out,
                            ld_out, /*store4=*/0, scales_out, ws, STATIC_SCRATCH_BYTES, (hipStream_t)hip_stream, who);
}
