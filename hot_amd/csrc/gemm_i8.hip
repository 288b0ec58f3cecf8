// gemm_i8: C[M,N] = A[M,K] . B[N,K]^T on integer codes with the gfx950 INT8
// matrix cores (v_mfma_i32_32x32x32_i8), fused dequantisation epilogue.
//
// Replaces CutlassSgemmNN_int4 / CutlassSgemmNN_int8 and the separate
// dequantize_cuda(_per_token)_kernel passes of the reference op
// (cuda_measure/HLQ_backward_kernel.cu:181-280,309-384,386-450); operand
// contract as there: A [M,K] and B [N,K] both K-major, int32 accumulation.
// Epilogue numerics follow utils/quant_matmul.py:288-290,322-324,343-344:
//   out = ((float(acc) * s_a) * s_b) * post_scale.
//
// gfx950 has no INT4 MFMA.  Packed INT4 operands stay packed in HBM and are
// expanded to int8 while the tile is staged into LDS: nibble v becomes the
// byte (v << 4), whose two's-complement value is 16 v, so no sign-extension
// arithmetic is needed; the accumulator is then 256 x the true one and is
// shifted back (exactly) in the epilogue.  Even and odd elements of each
// 32-code group land in separate 16-byte LDS slots for both operands alike,
// which permutes K consistently and leaves every dot product unchanged.
//
// Tiling: 256 threads = 2x2 waves; each wave owns (32 WM) x (32 WN) outputs as
// WM x WN MFMA tiles; K advances 128 codes per stage with the next stage's
// global loads in flight during the MFMAs (double-buffered LDS).
#include <mutex>
#include <type_traits>
#include <utility>

#include "hot_device.h"
#include "hot_host.h"

namespace hot {

constexpr int G_THREADS = 256;
constexpr int G_BK = 128;            // int8 bytes of K per stage in LDS
constexpr int G_PITCH = G_BK + 16;   // LDS row pitch: 16-byte reads by 8 consecutive rows hit 32 distinct banks

struct GemmArgs {
  const uint8_t* A;
  const uint8_t* B;
  int64_t lda, ldb;  // bytes
  int64_t M, N;
  int32_t ktiles;    // stages of G_BK codes
  const float* scale_a;
  const float* scale_b;
  float post_scale;
  int32_t a_per_row;
  void* out;
  int64_t ldo;
  const void* bias;  // 16-bit floating operands only (BITS = 16): NULL or N elements of the output type, added per column
  int32_t* acc_out;
  int32_t tiles_m, tiles_n;
  int32_t group_m;   // tile rows per group of the launch order (tile_of)
  int32_t vec_out;   // out and ldo allow aligned four-element stores
  int32_t vec16;     // out and its row pitch are 16-byte aligned (staged epilogue)
  int32_t splits;    // K is cut into this many ranges, one workgroup each (1 = no split)
  v4i* partials;     // [tile][range][wave][fragment quad][lane]: raw accumulators of the ranges
  // K groups (gemm_i8_grouped_kernel; 3-D activations: a group is a sample with steps of its own).
  // The integer sums of every group are dequantised with the group's steps and added, in group
  // order, to fp32 accumulators:
  //   out = (sum over groups of (float(acc_g) * sa_g[row or 0]) * sb_g) * post_scale.
  // With gsplits > 1 the groups are cut into gsplits contiguous ranges, one workgroup each; every
  // range leaves its fp32 sum in gpart and a second kernel adds the ranges in order.
  int32_t groups;
  int32_t group_stages;     // 128-byte stages per group
  int32_t gsplits, gper;    // ranges and groups per range
  const float* gscale_a;    // [groups] or, with a_per_row, [groups][M]
  const float* gscale_b;    // [groups]
  float* gpart;             // [gsplits][M][ldp] fp32
  int64_t ldp;
};

// Workgroup -> tile.  Hardware deals consecutive workgroup ids round-robin to the 8 XCDs, each with
// its own L2.  XCD x takes a contiguous chunk of the launch order, and the launch order walks the
// tile grid in groups of group_m tile rows, row index fastest inside a group, so the workgroups that
// are resident in one XCD at the same time form a compact block of tiles: they stream few distinct
// A and B row panels, and most of their loads hit in that XCD's L2.
// Position of workgroup `wg` in a launch order of `total` units in which XCD x (= wg % 8) takes the
// x-th contiguous chunk.
__device__ __forceinline__ int xcd_chunk_position(int total, int wg) {
  const int x = wg & 7, idx = wg >> 3;
  const int q = total >> 3, rem = total & 7;
  return x * q + (x < rem ? x : rem) + idx;
}

// Tile of position t in the grouped walk of the tile grid.
__device__ __forceinline__ void grouped_tile(const GemmArgs& g, int t, int& tm, int& tn) {
  const int per_group = g.group_m * g.tiles_n;
  const int grp = t / per_group, j = t - grp * per_group;
  const int rows = min(g.group_m, g.tiles_m - grp * g.group_m);
  tm = grp * g.group_m + j % rows;
  tn = j / rows;
}

__device__ __forceinline__ void tile_of(const GemmArgs& g, int wg, int& tm, int& tn) {
  const int total = g.tiles_m * g.tiles_n;
  const int t = xcd_chunk_position(total, wg);
  const int per_group = g.group_m * g.tiles_n;
  const int grp = t / per_group, j = t - grp * per_group;
  const int rows = min(g.group_m, g.tiles_m - grp * g.group_m);
  tm = grp * g.group_m + j % rows;
  tn = j / rows;
}

// Rows per group: about the square root of the tiles one XCD holds at a time.
static int pick_group_m(int tiles_m, int tiles_n, int wgs_per_cu) {
  const int64_t total = (int64_t)tiles_m * tiles_n;
  int64_t conc = total / 8 < 32 * wgs_per_cu ? total / 8 : 32 * wgs_per_cu;
  if (conc < 1) conc = 1;
  int gm = 1;
  while ((int64_t)(gm + 1) * (gm + 1) <= conc) ++gm;
  if (gm > tiles_m) gm = tiles_m;
  return gm;
}


// Fused dequantisation epilogue, shared by both kernels.  The MFMAs are issued with the operands
// swapped (B fragment first), so a 32x32 accumulator tile holds the TRANSPOSED product: lane l owns
// output row l % 32 and, in registers 4 q .. 4 q + 3, the four adjacent output columns
// 8 q + 4 (l / 32) .. + 3.  Each lane therefore stores four adjacent outputs at a time (8 bytes of
// bf16 / f16, 16 bytes of fp32), and lanes l and l + 32 fill neighbouring quads of one row.
template <typename OutT> struct Quad;
template <> struct Quad<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct Quad<bf16_t> { typedef uint16_t type __attribute__((ext_vector_type(4))); };
template <> struct Quad<f16_t> { typedef _Float16 type __attribute__((ext_vector_type(4))); };
template <typename OutT> __device__ __forceinline__ void quad_set(typename Quad<OutT>::type& q, int t, float v);
template <> __device__ __forceinline__ void quad_set<float>(Quad<float>::type& q, int t, float v) { q[t] = v; }
template <> __device__ __forceinline__ void quad_set<bf16_t>(Quad<bf16_t>::type& q, int t, float v) { q[t] = f32_to_bf16_rne(v); }
template <> __device__ __forceinline__ void quad_set<f16_t>(Quad<f16_t>::type& q, int t, float v) { q[t] = (_Float16)v; }

// The quantisation steps of this lane's output rows; loaded before the K loop so that the loads'
// latency is hidden behind it.
template <int WM>
__device__ __forceinline__ void load_row_scales(const GemmArgs& g, int64_t row_base, int lane, float (&sa_row)[WM]) {
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int64_t row = row_base + i * 32 + (lane & 31);
    sa_row[i] = g.a_per_row ? g.scale_a[row < g.M ? row : g.M - 1] : g.scale_a[0];
  }
}

// Output value of one accumulator register.  Integer codes: ((float(acc) * s_a) * s_b) * post_scale
// (packed INT4 accumulates 256 x the product).  BITS = 16 (bf16 operands): the register holds the
// fp32 sum itself, and `bias` (the column's bias, 0 without one) is added.
template <int BITS>
__device__ __forceinline__ float acc_value(int a, float sa, float sb, float post, float bias) {
  if constexpr (BITS == 16) return __builtin_bit_cast(float, a) + bias;
  if constexpr (BITS == 4) a >>= 8;
  return (((float)a * sa) * sb) * post;
}
template <typename OutT> __device__ __forceinline__ float bias_at(const void* bias, int64_t col);
template <> __device__ __forceinline__ float bias_at<float>(const void* bias, int64_t col) { return bias ? reinterpret_cast<const float*>(bias)[col] : 0.f; }
template <> __device__ __forceinline__ float bias_at<bf16_t>(const void* bias, int64_t col) {
  return bias ? as_f((uint32_t)reinterpret_cast<const uint16_t*>(bias)[col] << 16) : 0.f;
}
template <> __device__ __forceinline__ float bias_at<f16_t>(const void* bias, int64_t col) {
  return bias ? (float)reinterpret_cast<const _Float16*>(bias)[col] : 0.f;
}

template <int WM, int WN, int BITS, typename OutT>
__device__ __forceinline__ void gemm_epilogue(const v16i (&acc)[WM][WN], const GemmArgs& g, int64_t row_base,
                                              int64_t col_base, int lane, const float (&sa_row)[WM], float sb) {
  OutT* out = reinterpret_cast<OutT*>(g.out);
  const int half = lane >> 5;
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int64_t row = row_base + i * 32 + (lane & 31);
    if (row >= g.M) continue;
    const float sa = sa_row[i];
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t col = col_base + j * 32 + 8 * q + 4 * half;
        if (col >= g.N) continue;
        int a[4];
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          a[t] = acc[i][j][4 * q + t];
          if constexpr (BITS == 16) bv[t] = col + t < g.N ? bias_at<OutT>(g.bias, col + t) : 0.f;
        }
        if (g.acc_out) {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (col + t < g.N) g.acc_out[row * g.N + col + t] = BITS == 4 ? a[t] >> 8 : a[t];
        }
        if (g.vec_out && col + 3 < g.N) {
          typename Quad<OutT>::type v;
#pragma unroll
          for (int t = 0; t < 4; ++t) quad_set<OutT>(v, t, acc_value<BITS>(a[t], sa, sb, g.post_scale, bv[t]));
          *reinterpret_cast<typename Quad<OutT>::type*>(out + row * g.ldo + col) = v;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (col + t < g.N) store_scalar<OutT>(out + row * g.ldo + col + t, acc_value<BITS>(a[t], sa, sb, g.post_scale, bv[t]));
        }
      }
    }
  }
}

// Global -> register prefetch of one operand tile (ROWS x G_BK codes), and the
// register -> LDS store that expands packed INT4 on the way.
template <int ROWS, int BITS>
struct TileShape {
  static constexpr int GBYTES = G_BK * BITS / 8;        // bytes of one row of the stage in HBM
  static constexpr int CPR = GBYTES / 16;               // 16-byte chunks per row
  static constexpr int PER_THREAD = ROWS * CPR / G_THREADS;
};

template <int ROWS, int BITS, int PT>
__device__ __forceinline__ void tile_load(v4i (&r)[PT], const uint8_t* base, int64_t ld, int64_t row0,
                                          int64_t rows_total, int kt, int tid) {
  using S = TileShape<ROWS, BITS>;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int id = tid + i * G_THREADS;
    const int row = id / S::CPR, kc = id % S::CPR;
    int64_t gr = row0 + row;
    if (gr >= rows_total) gr = rows_total - 1;  // duplicate the last row; its outputs are never stored
    r[i] = *reinterpret_cast<const v4i*>(base + gr * ld + (int64_t)kt * S::GBYTES + kc * 16);
  }
}

template <int ROWS, int BITS, int PT>
__device__ __forceinline__ void tile_store(const v4i (&r)[PT], uint8_t* lds, int tid) {
  using S = TileShape<ROWS, BITS>;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int id = tid + i * G_THREADS;
    const int row = id / S::CPR, kc = id % S::CPR;
    if constexpr (BITS == 8) {
      *reinterpret_cast<v4i*>(lds + row * G_PITCH + kc * 16) = r[i];
    } else {
      // even elements (low nibbles) and odd elements (high nibbles), each as value << 4
      const v4i m = {(int)0xF0F0F0F0, (int)0xF0F0F0F0, (int)0xF0F0F0F0, (int)0xF0F0F0F0};
      const v4i ev = (r[i] << 4) & m, od = r[i] & m;
      *reinterpret_cast<v4i*>(lds + row * G_PITCH + kc * 32) = ev;
      *reinterpret_cast<v4i*>(lds + row * G_PITCH + kc * 32 + 16) = od;
    }
  }
}

template <int WM, int WN, int BITS, typename OutT>
__global__ void __launch_bounds__(G_THREADS) __attribute__((amdgpu_waves_per_eu(1, (WM * WN <= 4 ? 2 : 1))))
gemm_i8_kernel(const GemmArgs g) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  constexpr int A_BYTES = BM * G_PITCH, B_BYTES = BN * G_PITCH;
  extern __shared__ __align__(16) uint8_t lds[];
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;  // stage s: A at s * STAGE_BYTES, B right after

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  int tm, tn;
  tile_of(g, blockIdx.x, tm, tn);
  const int64_t row0 = (int64_t)tm * BM, col0 = (int64_t)tn * BN;
  float sa_row[WM];
  load_row_scales<WM>(g, row0 + wm * WM * 32, lane, sa_row);
  const float sb = g.scale_b[0];

  constexpr int PTA = TileShape<BM, BITS>::PER_THREAD, PTB = TileShape<BN, BITS>::PER_THREAD;
  v4i ra[PTA], rb[PTB];
  tile_load<BM, BITS, PTA>(ra, g.A, g.lda, row0, g.M, 0, tid);
  tile_load<BN, BITS, PTB>(rb, g.B, g.ldb, col0, g.N, 0, tid);

  v16i acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  tile_store<BM, BITS, PTA>(ra, lds, tid);
  tile_store<BN, BITS, PTB>(rb, lds + A_BYTES, tid);
  __syncthreads();

  const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
  for (int kt = 0; kt < g.ktiles; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < g.ktiles) {
      tile_load<BM, BITS, PTA>(ra, g.A, g.lda, row0, g.M, kt + 1, tid);
      tile_load<BN, BITS, PTB>(rb, g.B, g.ldb, col0, g.N, kt + 1, tid);
    }
    const uint8_t* pa = lds + cur * STAGE_BYTES + (wm * 32 * WM + frag_row) * G_PITCH + frag_k;
    const uint8_t* pb = lds + cur * STAGE_BYTES + A_BYTES + (wn * 32 * WN + frag_row) * G_PITCH + frag_k;
#pragma unroll
    for (int ks = 0; ks < G_BK / 32; ++ks) {
      v4i fa[WM], fb[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i) fa[i] = *reinterpret_cast<const v4i*>(pa + i * 32 * G_PITCH + ks * 32);
#pragma unroll
      for (int j = 0; j < WN; ++j) fb[j] = *reinterpret_cast<const v4i*>(pb + j * 32 * G_PITCH + ks * 32);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < g.ktiles) {
      tile_store<BM, BITS, PTA>(ra, lds + (cur ^ 1) * STAGE_BYTES, tid);
      tile_store<BN, BITS, PTB>(rb, lds + (cur ^ 1) * STAGE_BYTES + A_BYTES, tid);
    }
    __syncthreads();
  }

  gemm_epilogue<WM, WN, BITS, OutT>(acc, g, row0 + wm * WM * 32, col0 + wn * WN * 32, lane, sa_row, sb);
}

// Epilogue through LDS for tiles that lie fully inside the output: a wave turns one row of its
// fragments (32 output rows x WN * 32 columns) into output values, parks them row-major in a
// wave-private LDS area and writes them back out 16 bytes per lane along the rows, so every store
// instruction covers whole 128-byte lines (the direct epilogue hands the memory system 16-byte
// pieces of 32 different rows per instruction).  Wave-private: the only synchronisation is the
// wave's own LDS counter.  `area` must hold 32 * (WN * 32 * sizeof(OutT) + 16) bytes.
template <int WM, int WN, int BITS, typename OutT>
__device__ __forceinline__ void gemm_epilogue_staged(const v16i (&acc)[WM][WN], const GemmArgs& g, int64_t row_base,
                                                     int64_t col_base, int lane, const float (&sa_row)[WM], float sb,
                                                     uint8_t* area) {
  constexpr int ROWB = WN * 32 * (int)sizeof(OutT);     // bytes of one staged row
  constexpr int PITCH = ROWB + 16;
  constexpr int CPR = ROWB / 16;                        // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;                         // rows one wave-wide store covers
  typedef typename Quad<OutT>::type quad_t;
  OutT* out = reinterpret_cast<OutT*>(g.out);
  const int m = lane & 31, half = lane >> 5;
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const float sa = sa_row[i];
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        quad_t v;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          float bv = 0.f;     // (the staged epilogue runs on whole tiles only: every column exists)
          if constexpr (BITS == 16) bv = bias_at<OutT>(g.bias, col_base + j * 32 + 8 * q + 4 * half + t);
          quad_set<OutT>(v, t, acc_value<BITS>(acc[i][j][4 * q + t], sa, sb, g.post_scale, bv));
        }
        *reinterpret_cast<quad_t*>(area + m * PITCH + (j * 32 + 8 * q + 4 * half) * (int)sizeof(OutT)) = v;
      }
    __builtin_amdgcn_s_waitcnt(0xC07F);                 // lgkmcnt(0): the wave's LDS writes are done
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += RPI) {
      const int r = r0 + lane / CPR, c = lane % CPR;
      const v4i chunk = *reinterpret_cast<const v4i*>(area + r * PITCH + c * 16);
      *reinterpret_cast<v4i*>(reinterpret_cast<uint8_t*>(out + (row_base + i * 32 + r) * g.ldo + col_base) + c * 16) = chunk;
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);                 // reads done before the next fragment row overwrites
  }
}

// ---------------------------------------------------------------------------
// Pipelined variant: operand tiles travel HBM -> LDS without passing through
// registers (global_load_lds_dwordx4), four LDS stages deep, so that two
// K-tiles are always in flight behind the one being multiplied.  Packed INT4
// stays packed in LDS (half the LDS traffic) and is expanded to (v << 4) bytes
// right after the fragment read.
//
// LDS stage layout: rows of 64 bytes = four 16-byte slots; slot s of row r is
// stored at slot s ^ ((r >> 2) & 3), so the 16-byte fragment reads of 16
// consecutive rows (same logical slot) land in 16 different 16-byte bank groups
// of the 256-byte bank row.  A wave-wide DMA instruction fills one
// contiguous KiB (16 rows); lane l fills physical slot l of that KiB and so
// fetches row l >> 2, logical slot (l & 3) ^ ((l >> 4) & 3) from global memory.
//
// Each stage is its own __shared__ array and the K loop is unrolled by the
// stage count, so every LDS access names its stage statically; waits on the
// DMA are explicit (vmcnt) and the barrier carries no fence.
// ---------------------------------------------------------------------------

constexpr int P_ROWB = 64;  // bytes per row per stage

// s_waitcnt vmcnt(VM) alone (expcnt and lgkmcnt untouched); vmcnt is split over bits 3:0 and 15:14
template <int VM>
__device__ __forceinline__ void wait_dma() {
  __builtin_amdgcn_s_waitcnt((VM & 0xF) | ((VM >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// s_waitcnt vmcnt(VM) lgkmcnt(0): the DMA wait plus "this wave's LDS reads have all returned"
template <int VM>
__device__ __forceinline__ void wait_dma_lds() {
  __builtin_amdgcn_s_waitcnt((VM & 0xF) | ((VM >> 4) << 14) | (0x7 << 4) | (0x0 << 8));
}

// vmcnt wait that lets `tiles` (0 .. MAXT) groups of LPW loads stay in flight
template <int MAXT, int LPW, bool LDS = false>
__device__ __forceinline__ void wait_dma_upto(int tiles) {
  if constexpr (MAXT <= 0) {
    if constexpr (LDS) wait_dma_lds<0>(); else wait_dma<0>();
  } else {
    if (tiles >= MAXT) { if constexpr (LDS) wait_dma_lds<MAXT * LPW>(); else wait_dma<MAXT * LPW>(); }
    else wait_dma_upto<MAXT - 1, LPW, LDS>(tiles);
  }
}

template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) { static_for_impl(std::make_integer_sequence<int, N>{}, f); }

// One wave-wide 16-byte-per-lane load from global memory straight into LDS:
// lane l's 16 bytes land at lds_addr + 16 l.  `lds_addr` and `sbase` must be
// wave-uniform.  Written as inline assembly so that the explicit vmcnt waits
// of the pipeline below are the only ones: the compiler cannot tell which LDS
// stage a DMA targets and would otherwise drain all of them before every
// fragment read.
__device__ __forceinline__ void dma16(uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_offset(const uint8_t* p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t*)p;
}

template <int WM, int WN, int BITS, int S, typename OutT>
__global__ void __launch_bounds__(G_THREADS) __attribute__((amdgpu_waves_per_eu(1, (WM * WN <= 4 ? (S == 3 ? 3 : 2) : 1))))
gemm_i8_pipe_kernel(const GemmArgs g) {
  static_assert(S >= 3 && S * (WM + WN) * 4096 <= 160 * 1024, "three or more LDS stages within 160 KiB");
  constexpr int BM = 64 * WM, BN = 64 * WN;
  constexpr int STAGE_BYTES = (BM + BN) * P_ROWB;
  constexpr int LPW = (BM + BN) / 64;           // DMA instructions per wave per stage (KiB chunks / 4 waves)
  constexpr int GSTEP = P_ROWB;                 // global bytes per stage and row: 64 int8 codes or 128 packed INT4 codes
  __shared__ __attribute__((aligned(1024))) uint8_t ring[S * STAGE_BYTES];   // stage k at k * STAGE_BYTES

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_total = g.tiles_m * g.tiles_n;
  // Split launches order their (K range, tile) units range-major and give each XCD a contiguous
  // chunk: the workgroups sharing an L2 then work on ONE K range of a compact block of tiles, a
  // fraction of the operand bytes that all ranges of fewer tiles would touch.
  int split = 0, tile_id = (int)blockIdx.x, tm, tn;
  if (g.splits > 1) {
    const int u = xcd_chunk_position(tiles_total * g.splits, (int)blockIdx.x);
    split = u / tiles_total;
    tile_id = u - split * tiles_total;
    grouped_tile(g, tile_id, tm, tn);
  } else {
    tile_of(g, tile_id, tm, tn);
  }
  const int64_t row0 = (int64_t)tm * BM, col0 = (int64_t)tn * BN;
  // The steps of this lane's rows: loaded here, behind the K loop's latency, when registers allow;
  // the 256 x 256 tile has none to spare and loads them in the epilogue.
  constexpr bool EARLY_SCALES = WM * WN <= 4;
  float sa_row[WM];
  float sb = 0.f;
  if constexpr (EARLY_SCALES) {
    load_row_scales<WM>(g, row0 + wm * WM * 32, lane, sa_row);
    sb = g.scale_b[0];
  }

  // DMA instruction i of this wave fills KiB chunk 4 i + wave of the stage (A rows first, then B
  // rows; BM / 16 is a multiple of 4, so instruction i serves A for i < BM / 64 and B otherwise).
  uint32_t goff[LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int r = (4 * i + wave) * 16 + (lane >> 2);
    const int slot = (lane & 3) ^ ((lane >> 4) & 3);
    if (i < BM / 64) {
      int64_t gr = row0 + r;
      if (gr >= g.M) gr = g.M - 1;
      goff[i] = (uint32_t)(gr * g.lda + slot * 16);
    } else {
      int64_t gr = col0 + (r - BM);
      if (gr >= g.N) gr = g.N - 1;
      goff[i] = (uint32_t)(gr * g.ldb + slot * 16);
    }
  }
  // stages of this workgroup: its K range of the G_BK-code tiles, in 64-byte steps
  const int kt_all = g.ktiles * (G_BK / (BITS == 8 ? 64 : 128));
  const int kt_per = (kt_all + g.splits - 1) / g.splits;
  const int kt_begin = split * kt_per;
  const int KT = kt_all - kt_begin < kt_per ? kt_all - kt_begin : kt_per;
  auto issue = [&](const uint8_t* stage, int kt) {
    const uint32_t l0 = lds_offset(stage) + wave * 1024;
    const uint8_t* ga = g.A + (int64_t)(kt_begin + kt) * GSTEP;
    const uint8_t* gb = g.B + (int64_t)(kt_begin + kt) * GSTEP;
#pragma unroll
    for (int i = 0; i < LPW; ++i) dma16(l0 + i * 4096, goff[i], i < BM / 64 ? ga : gb);
  };

  v16i acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  // A stage holds two "rounds" of fragments.  In round d the lanes of half h (= lane / 32) read
  // slot 2 d + h of their row: 16 int8 codes (one MFMA) or 32 packed INT4 codes (two MFMAs: the
  // low nibbles, then the high nibbles; both operands alike, so every product pairs equal k).
  const int frow = lane & 31, fhalf = lane >> 5;
  const int sw = (frow >> 2) & 3;                              // same for rows r and r + 32 k
  const int offA = (wm * 32 * WM + frow) * P_ROWB, offB = (BM + wn * 32 * WN + frow) * P_ROWB;
  auto read_round = [&](const uint8_t* stage, int d, v4i (&fa)[WM], v4i (&fb)[WN]) {
    const int so = ((2 * d + fhalf) ^ sw) * 16;
#pragma unroll
    for (int i = 0; i < WM; ++i) fa[i] = *reinterpret_cast<const v4i*>(stage + offA + i * 32 * P_ROWB + so);
#pragma unroll
    for (int j = 0; j < WN; ++j) fb[j] = *reinterpret_cast<const v4i*>(stage + offB + j * 32 * P_ROWB + so);
  };
  auto mma_round = [&](const v4i (&fa)[WM], const v4i (&fb)[WN]) {
    if constexpr (BITS == 8) {
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0);
    } else {
      const v4i m = {(int)0xF0F0F0F0, (int)0xF0F0F0F0, (int)0xF0F0F0F0, (int)0xF0F0F0F0};
      v4i ea[WM], eb[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i) ea[i] = (fa[i] << 4) & m;
#pragma unroll
      for (int j = 0; j < WN; ++j) eb[j] = (fb[j] << 4) & m;
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(eb[j], ea[i], acc[i][j], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < WM; ++i) ea[i] = fa[i] & m;
#pragma unroll
      for (int j = 0; j < WN; ++j) eb[j] = fb[j] & m;
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(eb[j], ea[i], acc[i][j], 0, 0, 0);
    }
  };

  // prologue: S - 1 tiles in flight, tile 0 landed and visible, its first round in registers
  static_for<S - 1>([&](auto k) {
    if (k.value < KT) issue(ring + k.value * STAGE_BYTES, k.value);
  });
  wait_dma_upto<S - 2, LPW>((KT < S - 1 ? KT : S - 1) - 1);   // all but the youngest tiles: tile 0 is in
  __builtin_amdgcn_s_barrier();
  v4i a0[WM], b0[WN];
  read_round(ring, 0, a0, b0);

  // One K-tile.  `cur` holds tile kt, `nxt` tile kt+1 (in flight or landed), `fre` held tile kt-1
  // and receives tile kt+S-1.  The barrier sits in the middle of the tile, behind a block of MFMAs,
  // and the first fragments of tile kt+1 are fetched before the last MFMA block of tile kt starts,
  // so the matrix pipe keeps running across the tile boundary.
  auto ktile = [&](auto steady, const uint8_t* cur, const uint8_t* nxt, const uint8_t* fre, int kt) {
    // Scheduling: the fragment reads of the NEXT MFMA block are interleaved with the MFMAs of the
    // current one (one LDS read after every MPR MFMAs), so the reads issue while the matrix pipe
    // is busy instead of after the whole block; the fences keep the blocks themselves in order.
    constexpr int NREAD = WM + WN;                              // fragment reads per round
    constexpr int NMFMA = WM * WN * (BITS == 8 ? 1 : 2);        // MFMAs per round
    constexpr int MPR = NMFMA / NREAD > 0 ? NMFMA / NREAD : 1;  // MFMAs per read
    auto interleave = [&]() {
#pragma unroll
      for (int i = 0; i < NREAD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);    // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      // DS read
      }
      __builtin_amdgcn_sched_group_barrier(0x008, NMFMA - MPR * NREAD, 0);
    };
    v4i a1[WM], b1[WN];
    read_round(cur, 1, a1, b1);
    mma_round(a0, b0);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (decltype(steady)::value) {
      // steady state (kt + 3 < KT): straight-line code, so the compiler's LDS wait counts are exact
      wait_dma<(S - 3) * LPW>();                              // this wave's share of tile kt+1 has landed
      __builtin_amdgcn_s_barrier();                           // ... and everybody's; nobody reads tile kt-1 any more
      issue(fre, kt + S - 1);
      __builtin_amdgcn_sched_barrier(0);
      read_round(nxt, 0, a0, b0);
      mma_round(a1, b1);
      interleave();
    } else {
      if (kt + 1 < KT) {
        // tiles kt+2 .. min(kt+S-2, KT-1) may stay in flight
        wait_dma_upto<S - 3, LPW>((kt + S - 2 < KT - 1 ? kt + S - 2 : KT - 1) - (kt + 1));
        __builtin_amdgcn_s_barrier();
        if (kt + S - 1 < KT) issue(fre, kt + S - 1);
        read_round(nxt, 0, a0, b0);
      }
      __builtin_amdgcn_sched_barrier(0);
      mma_round(a1, b1);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // The loop is unrolled by the stage count, so every LDS address is a compile-time offset.
  auto rotation = [&](auto steady, int kt0) {
    static_for<S>([&](auto k) {
      constexpr int K = decltype(k)::value;
      if (decltype(steady)::value || kt0 + K < KT)
        ktile(steady, ring + K * STAGE_BYTES, ring + ((K + 1) % S) * STAGE_BYTES, ring + ((K + S - 1) % S) * STAGE_BYTES,
              kt0 + K);
    });
  };
  int kt0 = 0;
  for (; kt0 + 2 * S - 2 < KT; kt0 += S) rotation(std::true_type{}, kt0);   // every issue inside is in range
  for (; kt0 < KT; kt0 += S) rotation(std::false_type{}, kt0);

  if (WM * WN <= 4 && g.splits > 1) {     // only the 128 x 128 kernel is ever launched split
    // Split K: every range leaves its raw accumulators in the workspace (lane-major, so each store
    // is one contiguous KiB per wave); gemm_i8_reduce_kernel adds them up and runs the epilogue.
    constexpr int QUADS = WM * WN * 4;
    v4i* mine = g.partials + (((int64_t)tile_id * g.splits + split) * 4 + wave) * (QUADS * 64) + lane;
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          v4i c = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
          mine[((i * WN + j) * 4 + q) * 64] = c;
        }
    return;
  }

  if constexpr (!EARLY_SCALES) {
    load_row_scales<WM>(g, row0 + wm * WM * 32, lane, sa_row);
    sb = g.scale_b[0];
  }
  constexpr int AREA = 32 * (WN * 32 * (int)sizeof(OutT) + 16);
  if (4 * AREA <= S * STAGE_BYTES && g.vec16 && !g.acc_out && row0 + BM <= g.M && col0 + BN <= g.N) {
    __syncthreads();                                     // every wave is done with the ring
    gemm_epilogue_staged<WM, WN, BITS, OutT>(acc, g, row0 + wm * WM * 32, col0 + wn * WN * 32, lane, sa_row, sb,
                                             ring + wave * AREA);
    return;
  }
  gemm_epilogue<WM, WN, BITS, OutT>(acc, g, row0 + wm * WM * 32, col0 + wn * WN * 32, lane, sa_row, sb);
}

// ---------------------------------------------------------------------------
// Slot-scheduled variant.  Same data path as the pipelined kernel above (operand tiles HBM -> LDS by
// DMA through a ring of S stages, packed INT4 expanded after the fragment read), but the K loop is
// laid out by hand as a sequence of "slots", one MFMA each, fenced from one another, so that
// everything else rides in the shadow of the matrix pipe instead of between its blocks:
//   * the fragment reads of the NEXT round are issued in the first slots of the current round (in
//     the order the next round first uses them), so they have all returned when it starts;
//   * packed INT4: the low-nibble operands of the next round are expanded in the second half of the
//     current round, the high-nibble operands (in place) in the first half of their own round;
//   * the DMA instructions that refill a stage go out one per slot behind the barrier;
//   * a stage is refilled as soon as its second round is in registers (S - 1 tiles in flight).
// The wave grid is GM x GN (2 x 2, 1 x 4 or 4 x 1), a wave owns (32 WM) x (32 WN) outputs, so
// block tiles of any multiple of 32 rows exist (160 x 256 gives ViT-B's 12608 tokens x 768 one
// balanced round of 237 tiles on 256 CUs).  A stage holds (BM + BN) / 16 KiB chunks dealt round-
// robin to the four waves; when that is not a multiple of four the spare DMA slots fetch into a
// spare KiB, so that every wave issues the same number of loads and one vmcnt serves all.
// ---------------------------------------------------------------------------
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

template <int WM, int WN, int GM, int GN, int BITS, int S, int RB, typename OutT>
__global__ void __launch_bounds__(G_THREADS) __attribute__((amdgpu_waves_per_eu(1, (WM * WN <= 8 ? 2 : 1))))
gemm_i8_slot_kernel(const GemmArgs g) {
  static_assert(GM * GN == 4, "four waves");
  static_assert(RB == 64 || RB == 128, "stage rows of 64 or 128 bytes");
  constexpr int BM = 32 * WM * GM, BN = 32 * WN * GN;
  constexpr int SPR = RB / 16;                      // 16-byte slots per stage row
  constexpr int RPC = 1024 / RB;                    // rows per KiB chunk (one DMA instruction)
  constexpr int RPS = RB / 32;                      // rounds per stage: a round consumes 32 bytes of every row
  constexpr int ROWS = BM + BN, CHUNKS = ROWS / RPC, LPW = (CHUNKS + 3) / 4;
  constexpr bool SPARE = LPW * 4 != CHUNKS;
  constexpr int STAGE_BYTES = ROWS * RB;
  constexpr int RING_BYTES = S * STAGE_BYTES + (SPARE ? 1024 : 0);
  static_assert(S >= 2 && RING_BYTES <= 160 * 1024, "two or more LDS stages within 160 KiB");
  constexpr int NF = WM * WN;                       // accumulator fragments per wave
  constexpr int NM = NF * (BITS == 4 ? 2 : 1);      // MFMAs (slots) per round
  constexpr int NR = WM + WN;                       // fragment reads per round
  constexpr int H = NM / 2;                         // slots per half round
  constexpr int DPS = (LPW + NM - 1) / NM;          // DMA instructions per slot of the refilling round
  constexpr int RPSL = (NR + NM - 1) / NM;          // fragment reads per slot (1 unless NR > NM)
  static_assert(NR <= H || BITS != 4, "the reads of a round fit the first half of the round before");
  __shared__ __attribute__((aligned(1024))) uint8_t ring[RING_BYTES];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / GN, wn = wave % GN;
  int tm, tn;
  tile_of(g, (int)blockIdx.x, tm, tn);
  const int64_t row0 = (int64_t)tm * BM, col0 = (int64_t)tn * BN;
  constexpr bool EARLY_SCALES = NF <= 4 && BITS != 16;
  float sa_row[WM];
  float sb = 0.f;
  if constexpr (EARLY_SCALES) {
    load_row_scales<WM>(g, row0 + wm * WM * 32, lane, sa_row);
    sb = g.scale_b[0];
  }
  if constexpr (BITS == 16) {
#pragma unroll
    for (int i = 0; i < WM; ++i) sa_row[i] = 1.f;
  }

  // LDS stage layout: rows of RB bytes = SPR slots of 16 bytes; logical slot s of row r sits at
  // physical slot s ^ swz(r), swz(r) = (r >> 2) & 3 for 64-byte rows, (r >> 1) & 7 for 128-byte
  // rows: the fragment reads of 16 consecutive rows (same logical slot) then fall into 16 different
  // 16-byte bank groups.  DMA instruction i of this wave fills KiB chunk c = 4 i + wave of the
  // stage: rows RPC c .. RPC c + RPC - 1 (A rows first, then B rows); lane l fills physical slot
  // l % SPR of row l / SPR of the chunk.  Chunks past the end of the stage go to the spare KiB.
  uint32_t goff[LPW], ldst[LPW];
  uint32_t is_b = 0;                                // bit i: instruction i reads B
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    int c = 4 * i + wave;
    const bool spare = SPARE && c >= CHUNKS;
    ldst[i] = spare ? (uint32_t)(S * STAGE_BYTES) : (uint32_t)c * 1024u;
    if (spare) c = 0;
    const int r = c * RPC + lane / SPR;
    const int swz = RB == 64 ? (r >> 2) & 3 : (r >> 1) & 7;
    const int slot = (lane % SPR) ^ swz;
    if (c * RPC < BM) {
      int64_t gr = row0 + r;
      if (gr >= g.M) gr = g.M - 1;
      goff[i] = (uint32_t)(gr * g.lda + slot * 16);
    } else {
      int64_t gr = col0 + (r - BM);
      if (gr >= g.N) gr = g.N - 1;
      goff[i] = (uint32_t)(gr * g.ldb + slot * 16);
      is_b |= 1u << i;
    }
  }
  is_b = __builtin_amdgcn_readfirstlane(is_b);
  const uint32_t ring0 = lds_offset(ring);
  const int KT = g.ktiles * (G_BK * BITS / 8) / RB;               // stages of RB bytes per row
  // (copies in registers: selecting between the two kernel arguments by a run-time bit would reload
  // the pointer from the argument segment at every DMA instruction, and wait for it)
  const uint8_t* a_base = g.A;
  const uint8_t* b_base = g.B;
  asm volatile("" : "+s"(a_base), "+s"(b_base));
  auto dma_one = [&](int stage_off, int kt, int i) {
    // (wave-uniform by construction; said explicitly, since the instruction takes it in scalar registers)
    const uint64_t b64 = (uint64_t)(uintptr_t)(((is_b >> i) & 1u ? b_base : a_base) + (int64_t)kt * RB);
    // (the builtin returns a signed int: both halves go through uint32_t, or a low half with its top
    // bit set would sign-extend over the high half)
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b64 >> 32));
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b64);
    const uint8_t* base = reinterpret_cast<const uint8_t*>(((uint64_t)b_hi << 32) | (uint64_t)b_lo);
    const bool spare = SPARE && ldst[i] == (uint32_t)(S * STAGE_BYTES);
    dma16(ring0 + (spare ? 0u : (uint32_t)stage_off) + ldst[i], goff[i], base);
  };

  v16i acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  // Fragments of two consecutive rounds: fr[p][t], p = parity of the round within its stage, t in the
  // order of first use by the MFMAs (A fragment 0, the WN B fragments, then A fragments 1 .. WM - 1).
  // Packed INT4: lo[p][t] holds the low-nibble operands, fr[p][t] turns into the high-nibble operands
  // in place.  In round d of a stage the lanes of half h (= lane / 32) read logical slot 2 d + h of
  // their row: 16 int8 codes (one MFMA) or 32 packed INT4 codes (two MFMAs: the low nibbles, then the
  // high nibbles; both operands alike, so every product pairs equal k).
  v4i fr[2][NR], lo[2][BITS == 4 ? NR : 1];
  const int frow = lane & 31, fhalf = lane >> 5;
  const int sw = RB == 64 ? (frow >> 2) & 3 : (frow >> 1) & 7;     // same for rows r and r + 32 k
  const int offA = (wm * 32 * WM + frow) * RB, offB = (BM + wn * 32 * WN + frow) * RB;
  auto frag_off = [&](int t) {            // byte offset of fragment t within a stage, without the slot
    return t == 0 ? offA : (t <= WN ? offB + (t - 1) * 32 * RB : offA + (t - WN) * 32 * RB);
  };
  auto read_frag = [&](const uint8_t* stage, int d, int t) {
    const int so = ((2 * d + fhalf) ^ sw) * 16;
    fr[d & 1][t] = *reinterpret_cast<const v4i*>(stage + frag_off(t) + so);
  };
  auto a_of = [](int i) { return i == 0 ? 0 : WN + i; };   // fragment index of A fragment i
  auto b_of = [](int j) { return 1 + j; };
  // MFMA m of a round of parity p
  auto mfma_slot = [&](int p, int m) {
    const int mm = m % NF, i = mm / WN, j = mm % WN;
    if constexpr (BITS == 16) {
      // bf16 operands: the same 16 bytes per lane are eight bf16 of K, the accumulator registers hold fp32
      acc[i][j] = __builtin_bit_cast(v16i, __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                               __builtin_bit_cast(v8bf, fr[p][b_of(j)]), __builtin_bit_cast(v8bf, fr[p][a_of(i)]),
                                               __builtin_bit_cast(v16f, acc[i][j]), 0, 0, 0));
    } else if constexpr (BITS == 8) {
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[p][b_of(j)], fr[p][a_of(i)], acc[i][j], 0, 0, 0);
    } else {
      if (m < NF) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(lo[p][b_of(j)], lo[p][a_of(i)], acc[i][j], 0, 0, 0);
      else acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[p][b_of(j)], fr[p][a_of(i)], acc[i][j], 0, 0, 0);
    }
  };
  // dword items [e0, e1) of the expansions of the round of parity p: e = 4 t + dword
  auto expand_lo = [&](int p, int e0, int e1) {
#pragma unroll
    for (int e = e0; e < e1 && e < 4 * NR; ++e) lo[p][e >> 2][e & 3] = (fr[p][e >> 2][e & 3] << 4) & (int)0xF0F0F0F0;
  };
  auto expand_hi = [&](int p, int e0, int e1) {
#pragma unroll
    for (int e = e0; e < e1 && e < 4 * NR; ++e) fr[p][e >> 2][e & 3] &= (int)0xF0F0F0F0;
  };
  constexpr int EPS_ = BITS == 4 ? (4 * NR + H - 1) / H : 0;     // expansion items per slot of a half round

  // prologue: S tiles in flight, tile 0 landed and visible, its first round in registers
  static_for<S>([&](auto k) {
    if (k.value < KT) {
#pragma unroll
      for (int i = 0; i < LPW; ++i) dma_one(k.value * STAGE_BYTES, k.value, i);
    }
  });
  wait_dma_upto<S - 1, LPW>((KT < S ? KT : S) - 1);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int t = 0; t < NR; ++t) read_frag(ring, 0, t);
  if constexpr (BITS == 4) expand_lo(0, 0, 4 * NR);
  __builtin_amdgcn_sched_barrier(0);

  // One K tile in stage `cur` (tile kt + 1 in `nxt`).  `steady`: every predicate below is true.
  auto ktile = [&](auto steady, auto cur_off, auto nxt_off, int kt) {
    constexpr bool ST = decltype(steady)::value;
    constexpr int CUR = decltype(cur_off)::value, NXT = decltype(nxt_off)::value;
    const uint8_t* cur = ring + CUR;
    const uint8_t* nxt = ring + NXT;
    const bool more = ST || kt + 1 < KT;        // there is a tile kt + 1
    const bool refill = ST || kt + S < KT;      // ... and a tile kt + S to fetch into this stage
    static_for<RPS>([&](auto rc) {
      constexpr int r = decltype(rc)::value, p = r & 1;
      constexpr bool LAST = r == RPS - 1;
      if constexpr (LAST) {
        if (more) {
          // tile kt + 1 has landed (this wave's share) and this wave's reads of the stage are in ...
          if constexpr (ST) wait_dma_lds<(S - 2) * LPW>();
          else wait_dma_upto<S - 2, LPW, true>((kt + S - 1 < KT - 1 ? kt + S - 1 : KT - 1) - (kt + 1));
          __builtin_amdgcn_s_barrier();         // ... and everybody's: tile kt + 1 is visible, stage `cur` is free
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      // a round: reads of the next round (of this stage, or round 0 of the next tile), the refill of
      // this stage behind the barrier; INT4: high nibbles of this round, then low nibbles of the next
      static_for<NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        if constexpr (LAST) {
#pragma unroll
          for (int i = m * DPS; i < (m + 1) * DPS && i < LPW; ++i)
            if (refill) dma_one(CUR, kt + S, i);
        }
        // fragment reads of the next round: one per slot from the first slot on, or, when a wave owns
        // fewer MFMAs than fragments (tiles of one fragment row or column per wave), RPSL per slot
        static_for<RPSL>([&](auto tc) {
          constexpr int t = m * RPSL + decltype(tc)::value;
          if constexpr (t < NR) {
            if constexpr (!LAST) read_frag(cur, r + 1, t);
            else if (more) read_frag(nxt, 0, t);
          }
        });
        if constexpr (BITS == 4) {
          if constexpr (m < H) expand_hi(p, m * EPS_, (m + 1) * EPS_);
          else if (!LAST || more) expand_lo(p ^ 1, (m - H) * EPS_, (m - H + 1) * EPS_);
        }
        mfma_slot(p, m);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  auto rotation = [&](auto steady, int kt0) {
    static_for<S>([&](auto k) {
      constexpr int K = decltype(k)::value;
      if (decltype(steady)::value || kt0 + K < KT)
        ktile(steady, std::integral_constant<int, K * STAGE_BYTES>{}, std::integral_constant<int, ((K + 1) % S) * STAGE_BYTES>{},
              kt0 + K);
    });
  };
  int kt0 = 0;
  for (; kt0 + 2 * S - 1 < KT; kt0 += S) rotation(std::true_type{}, kt0);   // every tile inside has a tile kt + S
  for (; kt0 < KT; kt0 += S) rotation(std::false_type{}, kt0);

  if constexpr (!EARLY_SCALES && BITS != 16) {
    load_row_scales<WM>(g, row0 + wm * WM * 32, lane, sa_row);
    sb = g.scale_b[0];
  }
  constexpr int AREA = 32 * (WN * 32 * (int)sizeof(OutT) + 16);
  if (4 * AREA <= S * STAGE_BYTES && g.vec16 && !g.acc_out && row0 + BM <= g.M && col0 + BN <= g.N) {
    __syncthreads();                                     // every wave is done with the ring
    gemm_epilogue_staged<WM, WN, BITS, OutT>(acc, g, row0 + wm * WM * 32, col0 + wn * WN * 32, lane, sa_row, sb,
                                             ring + wave * AREA);
    return;
  }
  gemm_epilogue<WM, WN, BITS, OutT>(acc, g, row0 + wm * WM * 32, col0 + wn * WN * 32, lane, sa_row, sb);
}

// ---------------------------------------------------------------------------
// K groups with steps of their own (3-D activations: the K range of sample b holds the codes of
// sample b, and the reference dequantises every sample's product with that sample's steps before
// the sum over the batch, utils/quant_matmul.py:322-324 and the batch sum of autograd).
// INT8 operands, 128 x 128 tiles, the data path of the slot-scheduled kernel with 128-byte stage
// rows.  When a group ends, its integer sums are moved aside and, while the next group accumulates,
// converted, scaled twice (rounded after each product, as the reference's two multiplications are)
// and added to the fp32 accumulators, a few elements per MFMA slot, so the conversion rides in the
// shadow of the matrix pipe.  The first MFMA of a group takes a zero C operand, which replaces
// clearing the accumulators.  The ring stage is a run-time offset (a group may be any number of
// stages long).
// ---------------------------------------------------------------------------
template <typename OutT>
__global__ void __launch_bounds__(G_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1)))
gemm_i8_grouped_kernel(const GemmArgs g) {
  constexpr int WM = 2, WN = 2, GN = 2, S = 4, RB = 128;
  constexpr int BM = 128, BN = 128;
  constexpr int SPR = RB / 16, RPC = 1024 / RB, RPS = RB / 32;
  constexpr int ROWS = BM + BN, CHUNKS = ROWS / RPC, LPW = CHUNKS / 4;
  constexpr int STAGE_BYTES = ROWS * RB;
  constexpr int NF = WM * WN, NM = NF, NR = WM + WN;
  constexpr int DPS = (LPW + NM - 1) / NM;
  __shared__ __attribute__((aligned(1024))) uint8_t ring[S * STAGE_BYTES];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / GN, wn = wave % GN;
  const int tiles_total = g.tiles_m * g.tiles_n;
  int tm, tn, split = 0;
  {
    const int u = xcd_chunk_position(tiles_total * g.gsplits, (int)blockIdx.x);
    split = u / tiles_total;
    grouped_tile(g, u - split * tiles_total, tm, tn);
  }
  const int64_t row0 = (int64_t)tm * BM, col0 = (int64_t)tn * BN;
  const int g_lo = split * g.gper;
  const int g_hi = g_lo + g.gper < g.groups ? g_lo + g.gper : g.groups;
  const int gs = g.group_stages;
  const int KT = (g_hi - g_lo) * gs;                       // stages of this range
  const int64_t kbase = (int64_t)g_lo * gs * RB;           // byte offset of the range in every operand row

  uint32_t goff[LPW], ldst[LPW];
  uint32_t is_b = 0;
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int c = 4 * i + wave;
    ldst[i] = (uint32_t)c * 1024u;
    const int r = c * RPC + lane / SPR;
    const int slot = (lane % SPR) ^ ((r >> 1) & 7);
    if (c * RPC < BM) {
      int64_t gr = row0 + r;
      if (gr >= g.M) gr = g.M - 1;
      goff[i] = (uint32_t)(gr * g.lda + slot * 16);
    } else {
      int64_t gr = col0 + (r - BM);
      if (gr >= g.N) gr = g.N - 1;
      goff[i] = (uint32_t)(gr * g.ldb + slot * 16);
      is_b |= 1u << i;
    }
  }
  is_b = (uint32_t)__builtin_amdgcn_readfirstlane((int)is_b);
  const uint32_t ring0 = lds_offset(ring);
  const uint8_t* const a_base = g.A + kbase;
  const uint8_t* const b_base = g.B + kbase;
  auto dma_one = [&](uint32_t stage_off, int kt, int i) {
    const uint64_t b64 = (uint64_t)(uintptr_t)(((is_b >> i) & 1u ? b_base : a_base) + (int64_t)kt * RB);
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b64 >> 32));
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b64);
    dma16(ring0 + stage_off + ldst[i], goff[i], reinterpret_cast<const uint8_t*>(((uint64_t)b_hi << 32) | (uint64_t)b_lo));
  };

  // acc: integer sums of the group in progress; held: the finished sums of the group before it,
  // on their way into facc, the fp32 result
  v16i acc[WM][WN], held[WM][WN];
  v16f facc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      facc[i][j] = (v16f)(0.f);
#pragma unroll
      for (int e = 0; e < 16; ++e) { acc[i][j][e] = 0; held[i][j][e] = 0; }
    }
  // steps of the group being accumulated (c*) and of the held group (p*): all zero before the
  // first group, so that folding "the group before the first" adds nothing
  float csa[WM], psa[WM], csb = 0.f, psb = 0.f;
#pragma unroll
  for (int i = 0; i < WM; ++i) { csa[i] = 0.f; psa[i] = 0.f; }
  auto next_group_scales = [&](int gi) {
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      const int64_t row = row0 + wm * WM * 32 + i * 32 + (lane & 31);
      psa[i] = csa[i];
      csa[i] = g.a_per_row ? g.gscale_a[(int64_t)gi * g.M + (row < g.M ? row : g.M - 1)] : g.gscale_a[gi];
    }
    psb = csb;
    csb = g.gscale_b[gi];
  };

  v4i fr[2][NR];
  const int frow = lane & 31, fhalf = lane >> 5;
  const int sw = (frow >> 1) & 7;
  const int offA = (wm * 32 * WM + frow) * RB, offB = (BM + wn * 32 * WN + frow) * RB;
  auto frag_off = [&](int t) { return t == 0 ? offA : (t <= WN ? offB + (t - 1) * 32 * RB : offA + (t - WN) * 32 * RB); };
  auto read_frag = [&](const uint8_t* stage, int d, int t) {
    const int so = ((2 * d + fhalf) ^ sw) * 16;
    fr[d & 1][t] = *reinterpret_cast<const v4i*>(stage + frag_off(t) + so);
  };
  auto a_of = [](int i) { return i == 0 ? 0 : WN + i; };
  auto b_of = [](int j) { return 1 + j; };

  // prologue: up to S tiles in flight, tile 0 landed and visible, its first round in registers
#pragma unroll
  for (int k = 0; k < S; ++k)
    if (k < KT) {
#pragma unroll
      for (int i = 0; i < LPW; ++i) dma_one((uint32_t)(k * STAGE_BYTES), k, i);
    }
  wait_dma_upto<S - 1, LPW>((KT < S ? KT : S) - 1);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int t = 0; t < NR; ++t) read_frag(ring, 0, t);
  __builtin_amdgcn_sched_barrier(0);

  // One stage (16 slots: 4 rounds of 4 MFMAs).  FIRST: the stage opens a group: in round 0 the
  // slot of fragment f moves the finished sums of f aside (acc -> held) and restarts f with a zero
  // C operand.  The 64 held sums are folded into facc in QT "fold slots" (the slots of rounds 1-3
  // of the opening stage and, for groups of two stages or more, all slots of the second stage);
  // this stage owns the fold slots from Q0 on.  QT = 0: no folding in this stage.
  auto stage = [&](auto firstc, auto q0c, auto qtc, int kt) {
    constexpr bool FIRST = decltype(firstc)::value;
    constexpr int Q0 = decltype(q0c)::value, QT = decltype(qtc)::value;
    const uint32_t cur_off = (uint32_t)(kt & (S - 1)) * STAGE_BYTES;
    const uint8_t* cur = ring + cur_off;
    const uint8_t* nxt = ring + (uint32_t)((kt + 1) & (S - 1)) * STAGE_BYTES;
    const bool more = kt + 1 < KT, refill = kt + S < KT;
    static_for<RPS>([&](auto rc) {
      constexpr int r = decltype(rc)::value, p = r & 1;
      constexpr bool LAST = r == RPS - 1;
      if constexpr (LAST) {
        if (more) {
          wait_dma_upto<S - 2, LPW, true>((kt + S - 1 < KT - 1 ? kt + S - 1 : KT - 1) - (kt + 1));
          __builtin_amdgcn_s_barrier();
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      static_for<NM>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        if constexpr (LAST) {
#pragma unroll
          for (int i = m * DPS; i < (m + 1) * DPS && i < LPW; ++i)
            if (refill) dma_one(cur_off, kt + S, i);
        }
        if constexpr (!LAST) read_frag(cur, r + 1, m);
        else if (more) read_frag(nxt, 0, m);
        constexpr int q = FIRST ? Q0 + (r - 1) * NM + m : Q0 + r * NM + m;      // fold slot of this slot
        if constexpr (QT > 0 && (!FIRST || r >= 1) && q < QT) {
          // the product is rounded before it is added (no fused multiply-add): the sum over the
          // groups is the fp32 sum of the per-group results
#pragma clang fp contract(off)
          constexpr int E0 = q * 16 * NF / QT, E1 = (q + 1) * 16 * NF / QT;
#pragma unroll
          for (int e = E0; e < E1; ++e) {
            const int f = e / 16, k = e % 16, i = f / WN, j = f % WN;
            facc[i][j][k] += ((float)held[i][j][k] * psa[i]) * psb;
          }
        }
        const int i = m / WN, j = m % WN;
        if constexpr (FIRST && r == 0) {
          const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          held[i][j] = acc[i][j];
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[p][b_of(j)], fr[p][a_of(i)], zero, 0, 0, 0);
        } else {
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[p][b_of(j)], fr[p][a_of(i)], acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  using I0 = std::integral_constant<int, 0>;
  constexpr int Q1 = (RPS - 1) * NM, Q2 = Q1 + RPS * NM;     // fold slots of the opening stage, and of two stages
  int kt = 0;
  for (int gi = g_lo; gi < g_hi; ++gi) {
    next_group_scales(gi);
    if (gs == 1) {
      stage(std::true_type{}, I0{}, std::integral_constant<int, Q1>{}, kt++);
    } else {
      stage(std::true_type{}, I0{}, std::integral_constant<int, Q2>{}, kt++);
      stage(std::false_type{}, std::integral_constant<int, Q1>{}, std::integral_constant<int, Q2>{}, kt++);
      for (int s2 = 2; s2 < gs; ++s2) stage(std::false_type{}, I0{}, I0{}, kt++);
    }
  }
  // the last group's sums
  {
#pragma clang fp contract(off)
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) facc[i][j] += (__builtin_convertvector(acc[i][j], v16f) * csa[i]) * csb;
  }

  const int half = lane >> 5;
  if (g.gsplits > 1) {
    // this range's sum, unscaled; gemm_i8_grouped_reduce_kernel adds the ranges in order
    float* part = g.gpart + (int64_t)split * g.M * g.ldp;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      const int64_t row = row0 + wm * WM * 32 + i * 32 + (lane & 31);
      if (row >= g.M) continue;
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t col = col0 + wn * WN * 32 + j * 32 + 8 * q + 4 * half;
          if (col >= g.ldp) continue;          // ldp is N rounded up to 4: whole quads
          typedef float f4 __attribute__((ext_vector_type(4)));
          const f4 v = {facc[i][j][4 * q], facc[i][j][4 * q + 1], facc[i][j][4 * q + 2], facc[i][j][4 * q + 3]};
          *reinterpret_cast<f4*>(part + row * g.ldp + col) = v;
        }
    }
    return;
  }
  OutT* out = reinterpret_cast<OutT*>(g.out);
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int64_t row = row0 + wm * WM * 32 + i * 32 + (lane & 31);
    if (row >= g.M) continue;
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t col = col0 + wn * WN * 32 + j * 32 + 8 * q + 4 * half;
        if (col >= g.N) continue;
        if (g.vec_out && col + 3 < g.N) {
          typename Quad<OutT>::type v;
#pragma unroll
          for (int t = 0; t < 4; ++t) quad_set<OutT>(v, t, facc[i][j][4 * q + t] * g.post_scale);
          *reinterpret_cast<typename Quad<OutT>::type*>(out + row * g.ldo + col) = v;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (col + t < g.N) store_scalar<OutT>(out + row * g.ldo + col + t, facc[i][j][4 * q + t] * g.post_scale);
        }
      }
  }
}

// out = (part[0] + part[1] + ... in this order) * post_scale, one thread per four adjacent outputs
template <typename OutT>
__global__ void __launch_bounds__(256) gemm_i8_grouped_reduce_kernel(const GemmArgs g) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const int64_t quads_row = g.ldp / 4;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= g.M * quads_row) return;
  const int64_t row = id / quads_row, col = (id - row * quads_row) * 4;
  const float* p = g.gpart + row * g.ldp + col;
  f4 s = *reinterpret_cast<const f4*>(p);
  for (int k = 1; k < g.gsplits; ++k) s += *reinterpret_cast<const f4*>(p + (int64_t)k * g.M * g.ldp);
  OutT* out = reinterpret_cast<OutT*>(g.out);
  if (g.vec_out && col + 3 < g.N) {
    typename Quad<OutT>::type v;
#pragma unroll
    for (int t = 0; t < 4; ++t) quad_set<OutT>(v, t, s[t] * g.post_scale);
    *reinterpret_cast<typename Quad<OutT>::type*>(out + row * g.ldo + col) = v;
  } else {
#pragma unroll
    for (int t = 0; t < 4; ++t)
      if (col + t < g.N) store_scalar<OutT>(out + row * g.ldo + col + t, s[t] * g.post_scale);
  }
}

// Second kernel of a split-K product: one single-wave workgroup per 32 x 32 accumulator fragment,
// lane for lane the layout of the pipelined kernel, so each lane adds up the accumulators its twins
// left in the workspace (integer sums: any order gives the same result) and runs the same epilogue.
template <int WM, int WN, int BITS, typename OutT>
__global__ void __launch_bounds__(64) gemm_i8_reduce_kernel(const GemmArgs g) {
  constexpr int BM = 64 * WM, BN = 64 * WN, QUADS = WM * WN * 4, FRAGS = WM * WN;
  const int lane = threadIdx.x;
  const int frag = blockIdx.x % FRAGS, wave = (blockIdx.x / FRAGS) & 3, tile_id = blockIdx.x / (FRAGS * 4);
  const int fi = frag / WN, fj = frag % WN;
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  grouped_tile(g, tile_id, tm, tn);   // the numbering of the split launch
  const int64_t row0 = (int64_t)tm * BM + (wm * WM + fi) * 32, col0 = (int64_t)tn * BN + (wn * WN + fj) * 32;
  float sa_row[1];
  load_row_scales<1>(g, row0, lane, sa_row);
  const float sb = g.scale_b[0];
  v16i acc[1][1];
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[0][0][e] = 0;
  for (int s2 = 0; s2 < g.splits; ++s2) {
    const v4i* part = g.partials + (((int64_t)tile_id * g.splits + s2) * 4 + wave) * (QUADS * 64) + frag * 4 * 64 + lane;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v4i c = part[q * 64];
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[0][0][4 * q + t] += c[t];
    }
  }
  gemm_epilogue<1, 1, BITS, OutT>(acc, g, row0, col0, lane, sa_row, sb);
}

template <int WM, int WN, int BITS, int S, typename OutT>
static int launch_gemm_pipe(GemmArgs& g, hipStream_t st) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  g.tiles_m = (int)((g.M + BM - 1) / BM);
  g.tiles_n = (int)((g.N + BN - 1) / BN);
  g.group_m = pick_group_m(g.tiles_m, g.tiles_n, S == 3 && WM * WN <= 4 ? 3 : 1);
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  if (total > (1 << 30)) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: too many tiles");
  if (g.M * g.lda >= (1ll << 32) || g.N * g.ldb >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: operand larger than 4 GiB");
  hipLaunchKernelGGL((gemm_i8_pipe_kernel<WM, WN, BITS, S, OutT>), dim3((unsigned)(total * g.splits)), dim3(G_THREADS), 0, st, g);
  if (g.splits > 1) {
    if (int rc = check_launch("gemm_i8_pipe_kernel")) return rc;
    hipLaunchKernelGGL((gemm_i8_reduce_kernel<WM, WN, BITS, OutT>), dim3((unsigned)(total * 4 * WM * WN)), dim3(64), 0, st, g);
    return check_launch("gemm_i8_reduce_kernel");
  }
  return check_launch("gemm_i8_pipe_kernel");
}

template <int WM, int WN, int GM, int GN, int BITS, int S, int RB, typename OutT>
static int launch_gemm_slot(GemmArgs& g, hipStream_t st) {
  constexpr int BM = 32 * WM * GM, BN = 32 * WN * GN;
  g.tiles_m = (int)((g.M + BM - 1) / BM);
  g.tiles_n = (int)((g.N + BN - 1) / BN);
  g.group_m = pick_group_m(g.tiles_m, g.tiles_n, 1);
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  if (total > (1 << 30)) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: too many tiles");
  if (g.M * g.lda >= (1ll << 32) || g.N * g.ldb >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: operand larger than 4 GiB");
  if (((int64_t)g.ktiles * (G_BK * BITS / 8)) % RB) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: this kernel takes rows of a multiple of %d bytes", RB);
  hipLaunchKernelGGL((gemm_i8_slot_kernel<WM, WN, GM, GN, BITS, S, RB, OutT>), dim3((unsigned)total), dim3(G_THREADS), 0, st, g);
  return check_launch("gemm_i8_slot_kernel");
}

template <int WM, int WN, int BITS, typename OutT>
static int launch_gemm(GemmArgs& g, hipStream_t st) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  g.tiles_m = (int)((g.M + BM - 1) / BM);
  g.tiles_n = (int)((g.N + BN - 1) / BN);
  g.group_m = pick_group_m(g.tiles_m, g.tiles_n, 1);
  const size_t lds = (size_t)2 * (BM + BN) * G_PITCH;
  // one-time per instantiation; later calls only read the outcome
  static std::once_flag attr_once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(attr_once, [&] {
    attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_i8_kernel<WM, WN, BITS, OutT>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  });
  if (attr_err != hipSuccess) return check_hip(attr_err, "hipFuncSetAttribute(gemm_i8_kernel)");
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  if (total > (1 << 30)) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: too many tiles");
  hipLaunchKernelGGL((gemm_i8_kernel<WM, WN, BITS, OutT>), dim3((unsigned)total), dim3(G_THREADS), lds, st, g);
  return check_launch("gemm_i8_kernel");
}

// Split K when the 128 x 128 tiles cannot fill the chip: up to two workgroups per CU, at least 16
// stages of 64 bytes per range.
GemmSplit gemm_split_plan(int64_t M, int64_t N, int64_t K, int bits) {
  GemmSplit p; p.splits = 1; p.ws_bytes = 0;
  if (M <= 0 || N <= 0 || K <= 0) return p;
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  const int64_t stages = round_up(K, GEMM_KTILE) / (bits == 8 ? 64 : 128);
  int64_t sk = 1;
  if (tiles < 256) {
    sk = 512 / tiles;                        // about two workgroups per CU
    if (sk > stages / 16) sk = stages / 16;
    if (sk > 8) sk = 8;
  }
  if (sk > stages) sk = stages;
  if (sk < 2) return p;
  const int64_t per = (stages + sk - 1) / sk;
  sk = (stages + per - 1) / per;            // no empty range
  if (sk < 2) return p;
  p.splits = (int)sk;
  p.ws_bytes = (size_t)tiles * (size_t)sk * (128 * 128 * 4);
  return p;
}

// Which kernel a product takes.  Measured time of one round of up to 256 tiles (one per CU) as a
// function of K, in microseconds, on 8192..25216 x 768..11008 outputs with K = 768..11008:
//   128 x 128, pipelined, 2-3 workgroups per CU:  INT4 0.9 + 0.0037 K,   INT8 0.5 + 0.0052 K
//   128 x 128, slot-scheduled, one per CU:        INT4 1.0 + 0.0045 K,   INT8 1.5 + 0.0038 K
//   256 x 256, slot-scheduled:                    INT4 9 + 0.0108 K,     INT8 9 + 0.0122 K
//   256 x 256, pipelined:                         INT4 10 + 0.0131 K,    INT8 10 + 0.0136 K
//   160 x 256, slot-scheduled (INT4):             14.3 + 0.0064 K
// times the rounds a launch needs.  The 9-14 us of the large tiles are fill and epilogue that a lone
// workgroup per CU cannot overlap: INT8 operands take them from K of about 1100 on, packed INT4
// operands only from about 7000 on, and a product of exactly 256 large tiles beats 1024 small ones.
// Products of at most 256 small tiles with a long K take the slot-scheduled small kernel (one
// workgroup per CU, four 32 KiB stages) or, when they are few and a workspace is at hand, the
// split-K pair.  The slot-scheduled kernels stage 128 bytes of every row at a time and take rows of
// a multiple of 128 bytes only.  The DMA kernels address operands with 32-bit offsets; larger
// operands take the register-staged kernel.
int gemm_plan_impl(int64_t M, int64_t N, int64_t K, int bits, int64_t lda, int64_t ldb, size_t ws_bytes) {
  if (M <= 0 || N <= 0 || K <= 0 || (bits != 4 && bits != 8)) return HOT_GEMM_AUTO;
  if (M * lda >= (1ll << 32) || N * ldb >= (1ll << 32)) return HOT_GEMM_REG_128;
  const int64_t kpad = round_up(K, GEMM_KTILE);
  const bool rows128 = (kpad * bits / 8) % 128 == 0;
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  const int64_t big = ((M + 255) / 256) * ((N + 255) / 256);
  const int64_t mid = ((M + 159) / 160) * ((N + 255) / 256);
  const double k = (double)kpad;   // codes along K
  if (bits == 8 && rows128 && kpad >= 1024 && tiles <= 256) {
    // an INT8 product that leaves CUs idle at 128 x 128: the shortest tile (32, 64 or 96 rows of A against
    // 128 of B) that still gives every tile a CU of its own.  Measured at K = 7092 against 128 x 128
    // (and the split-K pair): 3072 x 768 25.5 against 29.3 us, 2304 x 768 20.3 / 27.2, 768 x 768 15.4 / 25.2
    // (21.2), 768 x 3072 24.1 / 28.3; a second round of tiles costs more than the longer tile.
    const int64_t tn = (N + 127) / 128;
    if (((M + 31) / 32) * tn <= 256) return HOT_GEMM_SLOT_32X128;
    if (((M + 63) / 64) * tn <= 256) return HOT_GEMM_SLOT_64X128;
    if (((M + 95) / 96) * tn <= 256) return HOT_GEMM_SLOT_96X128;
    return HOT_GEMM_SLOT_128;
  }
  const GemmSplit sp = gemm_split_plan(M, N, K, bits);
  if (sp.splits > 1 && ws_bytes >= sp.ws_bytes && !(rows128 && tiles >= 96)) return HOT_GEMM_DMA_128_SPLITK;
  if (tiles <= 256) return (rows128 && kpad >= 1024) ? HOT_GEMM_SLOT_128 : HOT_GEMM_DMA_128_S4;
  auto rounds = [](int64_t t) { return (double)((t + 255) / 256); };
  int best = bits == 4 ? HOT_GEMM_DMA_128_S3 : HOT_GEMM_DMA_128_S4;
  double t_best = (bits == 4 ? 0.9 + 0.0037 * k : 0.5 + 0.0052 * k) * rounds(tiles);
  if (big >= 256) {
    const double t = rows128 ? (9.0 + (bits == 4 ? 0.0108 : 0.0122) * k) * rounds(big)
                             : (10.0 + (bits == 4 ? 0.0131 : 0.0136) * k) * rounds(big);
    if (t < t_best) { t_best = t; best = rows128 ? HOT_GEMM_SLOT_256 : HOT_GEMM_DMA_256_S4; }
  }
  if (rows128 && bits == 4 && mid <= 256) {
    const double t = 14.3 + 0.0064 * k;
    if (t < t_best) { t_best = t; best = HOT_GEMM_SLOT_160X256; }
  }
  return best;
}

template <int BITS, typename OutT>
static int launch_variant(int variant, GemmArgs& g, hipStream_t st) {
  switch (variant) {
    case HOT_GEMM_DMA_128_S3: return launch_gemm_pipe<2, 2, BITS, 3, OutT>(g, st);
    case HOT_GEMM_DMA_128_S4: return launch_gemm_pipe<2, 2, BITS, 4, OutT>(g, st);
    case HOT_GEMM_DMA_256_S4: return launch_gemm_pipe<4, 4, BITS, 4, OutT>(g, st);
    case HOT_GEMM_DMA_128_SPLITK: return launch_gemm_pipe<2, 2, BITS, 3, OutT>(g, st);
    case HOT_GEMM_REG_128: return launch_gemm<2, 2, BITS, OutT>(g, st);
    case HOT_GEMM_SLOT_256: return launch_gemm_slot<4, 4, 2, 2, BITS, 2, 128, OutT>(g, st);
    case HOT_GEMM_SLOT_128: return launch_gemm_slot<2, 2, 2, 2, BITS, 4, 128, OutT>(g, st);
    case HOT_GEMM_SLOT_160X256: return launch_gemm_slot<5, 2, 1, 4, BITS, 2, 128, OutT>(g, st);
    case HOT_GEMM_SLOT_96X128:
      if constexpr (BITS == 8) return launch_gemm_slot<3, 1, 1, 4, 8, 4, 128, OutT>(g, st);
      else return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: the 96 x 128 kernel takes INT8 codes");
    case HOT_GEMM_SLOT_64X128:
      if constexpr (BITS == 8) return launch_gemm_slot<2, 1, 1, 4, 8, 4, 128, OutT>(g, st);
      else return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: the 64 x 128 kernel takes INT8 codes");
    case HOT_GEMM_SLOT_32X128:
      if constexpr (BITS == 8) return launch_gemm_slot<1, 1, 1, 4, 8, 4, 128, OutT>(g, st);
      else return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: the 32 x 128 kernel takes INT8 codes");
    default: return fail(HOT_ERR_INVALID, "hot_gemm_i8: unknown kernel variant %d", variant);
  }
}

template <int BITS>
static int dispatch_out(int out_dtype, int variant, GemmArgs& g, hipStream_t st) {
  switch (out_dtype) {
    case HOT_F32: return launch_variant<BITS, float>(variant, g, st);
    case HOT_BF16: return launch_variant<BITS, bf16_t>(variant, g, st);
    case HOT_F16: return launch_variant<BITS, f16_t>(variant, g, st);
    default: return fail(HOT_ERR_INVALID, "hot_gemm_i8: bad out dtype %d", out_dtype);
  }
}

int gemm_i8_impl(const void* A, int64_t lda, const void* B, int64_t ldb, int bits, int64_t M, int64_t N,
                 int64_t K, const float* scale_a, int a_per_row, const float* scale_b, float post_scale,
                 void* out, int out_dtype, int64_t ldo, int32_t* acc_out, hipStream_t st, void* split_ws,
                 size_t split_ws_bytes, int variant) {
  if (!A || !B || !scale_a || !scale_b || !out) return fail(HOT_ERR_INVALID, "hot_gemm_i8: null pointer");
  if (M < 0 || N < 0 || K <= 0) return fail(HOT_ERR_INVALID, "hot_gemm_i8: bad shape %lld x %lld x %lld", (long long)M, (long long)N, (long long)K);
  if (bits != 4 && bits != 8) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: bits=%d (4 or 8)", bits);
  const int64_t kpad = round_up(K, GEMM_KTILE);
  const int64_t need = kpad * bits / 8;
  if (lda < need || ldb < need || (lda & 15) || (ldb & 15))
    return fail(HOT_ERR_INVALID, "hot_gemm_i8: row pitches (%lld, %lld) must be multiples of 16 and >= %lld bytes", (long long)lda, (long long)ldb, (long long)need);
  if (((uintptr_t)A & 15) || ((uintptr_t)B & 15)) return fail(HOT_ERR_INVALID, "hot_gemm_i8: operands must be 16-byte aligned");
  if (ldo < N) return fail(HOT_ERR_INVALID, "hot_gemm_i8: ldo=%lld < N", (long long)ldo);
  if (bits == 4 && K > (int64_t)(0x7FFFFFFF / (112 * 112))) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: K too large for the scaled INT4 accumulator");
  if (bits == 8 && K > (int64_t)(0x7FFFFFFF / (127 * 127))) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: K too large for int32 accumulation");
  if (variant < HOT_GEMM_AUTO || variant >= HOT_GEMM_VARIANTS) return fail(HOT_ERR_INVALID, "hot_gemm_i8: unknown kernel variant %d", variant);
  if (M == 0 || N == 0) return HOT_OK;
  const size_t ws_have = split_ws ? split_ws_bytes : 0;
  if (variant == HOT_GEMM_AUTO) variant = gemm_plan_impl(M, N, K, bits, lda, ldb, ws_have);
  const bool small_ptrs = M * lda < (1ll << 32) && N * ldb < (1ll << 32);
  if (variant != HOT_GEMM_REG_128 && !small_ptrs)
    return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: operands of 4 GiB or more take the register-staged kernel only");
  GemmArgs g;
  g.A = (const uint8_t*)A; g.B = (const uint8_t*)B; g.lda = lda; g.ldb = ldb; g.M = M; g.N = N;
  g.ktiles = (int)(kpad / G_BK);
  g.scale_a = scale_a; g.scale_b = scale_b; g.post_scale = post_scale; g.a_per_row = a_per_row;
  g.out = out; g.ldo = ldo; g.acc_out = acc_out; g.bias = nullptr;
  g.vec_out = ((ldo & 3) == 0 && ((uintptr_t)out & 15) == 0) ? 1 : 0;
  g.vec16 = (((uintptr_t)out & 15) == 0 && ((ldo * (out_dtype == HOT_F32 ? 4 : 2)) & 15) == 0) ? 1 : 0;
  g.splits = 1; g.partials = nullptr;
  g.groups = 0; g.group_stages = 0; g.gsplits = 1; g.gper = 0; g.gscale_a = nullptr; g.gscale_b = nullptr; g.gpart = nullptr; g.ldp = 0;
  if (variant == HOT_GEMM_DMA_128_SPLITK) {
    const GemmSplit plan = gemm_split_plan(M, N, K, bits);
    if (plan.splits < 2) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: the split-K kernel needs a product of fewer than 256 tiles of 128 x 128 and a long K");
    if (ws_have < plan.ws_bytes) return fail(HOT_ERR_WORKSPACE, "hot_gemm_i8: split-K workspace of %zu bytes needed, %zu given", plan.ws_bytes, ws_have);
    if ((uintptr_t)split_ws & 15) return fail(HOT_ERR_INVALID, "hot_gemm_i8: workspace must be 16-byte aligned");
    g.splits = plan.splits;
    g.partials = (v4i*)split_ws;
  }
  return bits == 4 ? dispatch_out<4>(out_dtype, variant, g, st) : dispatch_out<8>(out_dtype, variant, g, st);
}

// out[M, N] = A[M, K] . B[N, K]^T (+ bias[N]) on bf16 operands, fp32 accumulation
// (v_mfma_f32_32x32x16_bf16), through the data path of the slot-scheduled integer kernels: a lane's 16
// bytes of a stage row are eight bf16 of K instead of sixteen codes, nothing else changes.  The plain
// linear layer y = x W^T + b of the forward pass (utils/quant_matmul.py:173-176, F.linear), built to
// measure this data path against the vendor library at the layer shapes.
int gemm_bf16_impl(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t M, int64_t N, int64_t K,
                   const void* bias, void* out, int out_dtype, int64_t ldo, hipStream_t st, int variant) {
  const char* who = "hot_gemm_bf16";
  if (!A || !B || !out) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (M < 0 || N < 0 || K <= 0) return fail(HOT_ERR_INVALID, "%s: bad shape %lld x %lld x %lld", who, (long long)M, (long long)N, (long long)K);
  if (K % G_BK) return fail(HOT_ERR_UNSUPPORTED, "%s: K=%lld must be a multiple of %d", who, (long long)K, G_BK);
  if (lda < 2 * K || ldb < 2 * K || (lda & 15) || (ldb & 15))
    return fail(HOT_ERR_INVALID, "%s: row pitches (%lld, %lld) are in bytes: multiples of 16, at least %lld", who, (long long)lda, (long long)ldb, (long long)(2 * K));
  if (((uintptr_t)A & 15) || ((uintptr_t)B & 15)) return fail(HOT_ERR_INVALID, "%s: operands must be 16-byte aligned", who);
  if (ldo < N) return fail(HOT_ERR_INVALID, "%s: ldo=%lld < N", who, (long long)ldo);
  if (M * lda >= (1ll << 32) || N * ldb >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "%s: operands of 4 GiB or more", who);
  if (M == 0 || N == 0) return HOT_OK;
  GemmArgs g;
  g.A = (const uint8_t*)A; g.B = (const uint8_t*)B; g.lda = lda; g.ldb = ldb; g.M = M; g.N = N;
  g.ktiles = (int)(K / G_BK);
  g.scale_a = nullptr; g.scale_b = nullptr; g.post_scale = 1.0f; g.a_per_row = 0;
  g.out = out; g.ldo = ldo; g.acc_out = nullptr; g.bias = bias;
  g.vec_out = ((ldo & 3) == 0 && ((uintptr_t)out & 15) == 0) ? 1 : 0;
  g.vec16 = (((uintptr_t)out & 15) == 0 && ((ldo * (out_dtype == HOT_F32 ? 4 : 2)) & 15) == 0) ? 1 : 0;
  g.splits = 1; g.partials = nullptr;
  g.groups = 0; g.group_stages = 0; g.gsplits = 1; g.gper = 0; g.gscale_a = nullptr; g.gscale_b = nullptr; g.gpart = nullptr; g.ldp = 0;
  if (variant == HOT_GEMM_AUTO) {
    // the 160 x 256 tile where it gives one balanced round (as for the integer products), else 256 x 256
    // while it fills the chip, else 128 x 128
    const int64_t t256 = ((M + 255) / 256) * ((N + 255) / 256);
    const int64_t t160 = ((M + 159) / 160) * ((N + 255) / 256);
    variant = (t160 <= 256 && t160 > t256) ? HOT_GEMM_SLOT_160X256 : (t256 >= 192 ? HOT_GEMM_SLOT_256 : HOT_GEMM_SLOT_128);
  }
#define HOT_BF16_CASE(OUT)                                                                                     \
  switch (variant) {                                                                                           \
    case HOT_GEMM_SLOT_256: return launch_gemm_slot<4, 4, 2, 2, 16, 2, 128, OUT>(g, st);                       \
    case HOT_GEMM_SLOT_128: return launch_gemm_slot<2, 2, 2, 2, 16, 4, 128, OUT>(g, st);                       \
    case HOT_GEMM_SLOT_160X256: return launch_gemm_slot<5, 2, 1, 4, 16, 2, 128, OUT>(g, st);                   \
    default: return fail(HOT_ERR_UNSUPPORTED, "%s: kernel variant %d (the slot-scheduled kernels only)", who, variant); \
  }
  switch (out_dtype) {
    case HOT_BF16: HOT_BF16_CASE(bf16_t)
    case HOT_F32: HOT_BF16_CASE(float)
    default: return fail(HOT_ERR_UNSUPPORTED, "%s: output type %d (bf16 or fp32)", who, out_dtype);
  }
#undef HOT_BF16_CASE
}

// INT8 product whose K dimension is `groups` samples of group_k codes each (a multiple of 128), every
// sample with steps of its own: out = (sum_g (float(acc_g) * sa[g][row or 0]) * sb[g]) * post_scale,
// the groups added in order in fp32.  128 x 128 tiles, slot-scheduled, one workgroup per tile.
// Ranges of groups a grouped product is cut into (a function of the shape alone, so that the order
// of the fp32 sum is reproducible: ranges of ceil(groups / ranges) consecutive groups, each summed in
// group order, the range sums added in range order).  One workgroup per tile and range occupies a
// CU; few tiles with many groups leave most of the 256 CUs idle unless the groups are shared out,
// and every range costs a round trip of the fp32 result.
int gemm_grouped_splits_impl(int64_t M, int64_t N, int groups, int64_t group_k) {
  if (M <= 0 || N <= 0 || groups <= 1 || group_k <= 0) return 1;
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  const double t_group = 2.0 * (double)group_k / 256.0;             // us per group and tile (measured: 128 groups of 256 codes in 260 us)
  const double t_part = (double)M * (double)N * 8.0 / 3.0e6;        // us per range: partial written and read
  int best = 1;
  double t_best = (double)((tiles + 255) / 256) * groups * t_group;
  const int smax = groups < 32 ? groups : 32;
  for (int sp = 2; sp <= smax; ++sp) {
    const int per = (groups + sp - 1) / sp;
    if ((sp - 1) * per >= groups) continue;                         // not a partition into sp non-empty ranges
    const double t = (double)((tiles * sp + 255) / 256) * per * t_group + sp * t_part + 3.0;
    if (t < t_best * 0.97) { t_best = t; best = sp; }
  }
  return best;
}

size_t gemm_grouped_workspace_bytes_impl(int64_t M, int64_t N, int groups, int64_t group_k) {
  const int sp = gemm_grouped_splits_impl(M, N, groups, group_k);
  return sp > 1 ? (size_t)sp * (size_t)M * (size_t)round_up(N, 4) * 4 : 0;
}

int gemm_i8_grouped_impl(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t M, int64_t N, int groups,
                         int64_t group_k, const float* scale_a, int a_per_row, const float* scale_b, float post_scale,
                         void* out, int out_dtype, int64_t ldo, void* workspace, size_t workspace_bytes, hipStream_t st) {
  const char* who = "hot_gemm_i8_grouped";
  if (!A || !B || !scale_a || !scale_b || !out) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (M < 0 || N < 0 || groups < 1 || group_k <= 0 || (group_k % 128)) return fail(HOT_ERR_INVALID, "%s: bad shape %lld x %lld, %d groups of %lld codes (a multiple of 128)", who, (long long)M, (long long)N, groups, (long long)group_k);
  const int64_t K = (int64_t)groups * group_k;
  if (lda < K || ldb < K || (lda & 15) || (ldb & 15)) return fail(HOT_ERR_INVALID, "%s: row pitches (%lld, %lld) must be multiples of 16 and >= %lld bytes", who, (long long)lda, (long long)ldb, (long long)K);
  if (((uintptr_t)A & 15) || ((uintptr_t)B & 15)) return fail(HOT_ERR_INVALID, "%s: operands must be 16-byte aligned", who);
  if (ldo < N) return fail(HOT_ERR_INVALID, "%s: ldo=%lld < N", who, (long long)ldo);
  if (group_k > (int64_t)(0x7FFFFFFF / (127 * 127))) return fail(HOT_ERR_UNSUPPORTED, "%s: group too long for int32 accumulation", who);
  if (M * lda >= (1ll << 32) || N * ldb >= (1ll << 32)) return fail(HOT_ERR_UNSUPPORTED, "%s: operand larger than 4 GiB", who);
  if (M == 0 || N == 0) return HOT_OK;
  GemmArgs g;
  g.A = (const uint8_t*)A; g.B = (const uint8_t*)B; g.lda = lda; g.ldb = ldb; g.M = M; g.N = N;
  g.ktiles = (int)(K / G_BK);
  g.scale_a = scale_a; g.scale_b = scale_b; g.post_scale = post_scale; g.a_per_row = a_per_row;
  g.out = out; g.ldo = ldo; g.acc_out = nullptr; g.bias = nullptr;
  g.vec_out = ((ldo & 3) == 0 && ((uintptr_t)out & 15) == 0) ? 1 : 0;
  g.vec16 = 0;
  g.splits = 1; g.partials = nullptr;
  g.groups = groups; g.group_stages = (int)(group_k / 128); g.gscale_a = scale_a; g.gscale_b = scale_b;
  g.gsplits = gemm_grouped_splits_impl(M, N, groups, group_k);
  g.gper = (groups + g.gsplits - 1) / g.gsplits;
  g.gpart = nullptr; g.ldp = round_up(N, 4);
  if (g.gsplits > 1) {
    const size_t need = gemm_grouped_workspace_bytes_impl(M, N, groups, group_k);
    if (!workspace || workspace_bytes < need) return fail(HOT_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
    if ((uintptr_t)workspace & 15) return fail(HOT_ERR_INVALID, "%s: workspace must be 16-byte aligned", who);
    g.gpart = (float*)workspace;
  }
  g.tiles_m = (int)((M + 127) / 128);
  g.tiles_n = (int)((N + 127) / 128);
  g.group_m = pick_group_m(g.tiles_m, g.tiles_n, 1);
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n * g.gsplits;
  if (total > (1 << 30)) return fail(HOT_ERR_UNSUPPORTED, "%s: too many tiles", who);
  const int64_t quads = M * (g.ldp / 4);
  const dim3 rgrid((unsigned)((quads + 255) / 256));
  switch (out_dtype) {
    case HOT_F32:
      hipLaunchKernelGGL(gemm_i8_grouped_kernel<float>, dim3((unsigned)total), dim3(G_THREADS), 0, st, g);
      if (g.gsplits > 1) hipLaunchKernelGGL(gemm_i8_grouped_reduce_kernel<float>, rgrid, dim3(256), 0, st, g);
      break;
    case HOT_BF16:
      hipLaunchKernelGGL(gemm_i8_grouped_kernel<bf16_t>, dim3((unsigned)total), dim3(G_THREADS), 0, st, g);
      if (g.gsplits > 1) hipLaunchKernelGGL(gemm_i8_grouped_reduce_kernel<bf16_t>, rgrid, dim3(256), 0, st, g);
      break;
    case HOT_F16:
      hipLaunchKernelGGL(gemm_i8_grouped_kernel<f16_t>, dim3((unsigned)total), dim3(G_THREADS), 0, st, g);
      if (g.gsplits > 1) hipLaunchKernelGGL(gemm_i8_grouped_reduce_kernel<f16_t>, rgrid, dim3(256), 0, st, g);
      break;
    default: return fail(HOT_ERR_INVALID, "%s: bad out dtype %d", who, out_dtype);
  }
  return check_launch("gemm_i8_grouped_kernel");
}

}  // namespace hot
