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
  int32_t* acc_out;
  int32_t tiles_m, tiles_n;
};

// Global -> register prefetch of one operand tile (ROWS x G_BK codes).
template <int ROWS, int BITS>
struct TileLoader {
  static constexpr int GBYTES = G_BK * BITS / 8;        // bytes of one row of the stage in HBM
  static constexpr int CPR = GBYTES / 16;               // 16-byte chunks per row
  static constexpr int PER_THREAD = ROWS * CPR / G_THREADS;
  uint4 r[PER_THREAD];

  __device__ __forceinline__ void load(const uint8_t* base, int64_t ld, int64_t row0, int64_t rows_total, int kt, int tid) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int id = tid + i * G_THREADS;
      const int row = id / CPR, kc = id % CPR;
      int64_t gr = row0 + row;
      if (gr >= rows_total) gr = rows_total - 1;  // duplicate the last row; its outputs are never stored
      r[i] = *reinterpret_cast<const uint4*>(base + gr * ld + (int64_t)kt * GBYTES + kc * 16);
    }
  }

  __device__ __forceinline__ void store(uint8_t* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int id = tid + i * G_THREADS;
      const int row = id / CPR, kc = id % CPR;
      if constexpr (BITS == 8) {
        *reinterpret_cast<uint4*>(lds + row * G_PITCH + kc * 16) = r[i];
      } else {
        uint4 ev, od;  // even elements (low nibbles) and odd elements (high nibbles), each as value << 4
        ev.x = (r[i].x << 4) & 0xF0F0F0F0u; od.x = r[i].x & 0xF0F0F0F0u;
        ev.y = (r[i].y << 4) & 0xF0F0F0F0u; od.y = r[i].y & 0xF0F0F0F0u;
        ev.z = (r[i].z << 4) & 0xF0F0F0F0u; od.z = r[i].z & 0xF0F0F0F0u;
        ev.w = (r[i].w << 4) & 0xF0F0F0F0u; od.w = r[i].w & 0xF0F0F0F0u;
        *reinterpret_cast<uint4*>(lds + row * G_PITCH + kc * 32) = ev;
        *reinterpret_cast<uint4*>(lds + row * G_PITCH + kc * 32 + 16) = od;
      }
    }
  }
};

template <int WM, int WN, int BITS, typename OutT>
__global__ void __launch_bounds__(G_THREADS) gemm_i8_kernel(const GemmArgs g) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  constexpr int A_BYTES = BM * G_PITCH, B_BYTES = BN * G_PITCH;
  extern __shared__ __align__(16) uint8_t lds[];
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;  // stage s: A at s * STAGE_BYTES, B right after

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // Workgroup -> tile.  Hardware deals consecutive workgroup ids round-robin
  // to the 8 XCDs; give each XCD a contiguous range of tiles (N fastest) so
  // the tiles sharing an A row panel meet in one L2.
  int tile;
  {
    const int total = g.tiles_m * g.tiles_n;
    const int wg = blockIdx.x;
    const int x = wg & 7, idx = wg >> 3;
    const int q = total >> 3, rem = total & 7;
    tile = x * q + (x < rem ? x : rem) + idx;
  }
  const int tm = tile / g.tiles_n, tn = tile % g.tiles_n;
  const int64_t row0 = (int64_t)tm * BM, col0 = (int64_t)tn * BN;

  TileLoader<BM, BITS> la;
  TileLoader<BN, BITS> lb;
  la.load(g.A, g.lda, row0, g.M, 0, tid);
  lb.load(g.B, g.ldb, col0, g.N, 0, tid);

  v16i acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  la.store(lds, tid);
  lb.store(lds + A_BYTES, tid);
  __syncthreads();

  const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
  for (int kt = 0; kt < g.ktiles; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < g.ktiles) {
      la.load(g.A, g.lda, row0, g.M, kt + 1, tid);
      lb.load(g.B, g.ldb, col0, g.N, kt + 1, tid);
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
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < g.ktiles) {
      la.store(lds + (cur ^ 1) * STAGE_BYTES, tid);
      lb.store(lds + (cur ^ 1) * STAGE_BYTES + A_BYTES, tid);
    }
    __syncthreads();
  }

  // Epilogue.  In a 32x32 accumulator tile lane l, register e holds
  // row 8 (e / 4) + 4 (l / 32) + (e % 4), column l % 32.
  const float sb = g.scale_b[0];
  const float sa0 = g.a_per_row ? 0.f : g.scale_a[0];
  OutT* out = reinterpret_cast<OutT*>(g.out);
#pragma unroll
  for (int i = 0; i < WM; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int64_t row = row0 + (wm * WM + i) * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
      if (row >= g.M) continue;
      const float sa = g.a_per_row ? g.scale_a[row] : sa0;
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const int64_t col = col0 + (wn * WN + j) * 32 + (lane & 31);
        if (col >= g.N) continue;
        int a = acc[i][j][e];
        if constexpr (BITS == 4) a >>= 8;
        if (g.acc_out) g.acc_out[row * g.N + col] = a;
        const float v = (((float)a * sa) * sb) * g.post_scale;
        store_scalar<OutT>(out + row * g.ldo + col, v);
      }
    }
  }
}

template <int WM, int WN, int BITS, typename OutT>
static int launch_gemm(GemmArgs& g, hipStream_t st) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  g.tiles_m = (int)((g.M + BM - 1) / BM);
  g.tiles_n = (int)((g.N + BN - 1) / BN);
  const size_t lds = (size_t)2 * (BM + BN) * G_PITCH;
  static bool attr_done = false;  // one-time, read-only afterwards
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_i8_kernel<WM, WN, BITS, OutT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return check_hip(e, "hipFuncSetAttribute(gemm_i8_kernel)");
    attr_done = true;
  }
  const int64_t total = (int64_t)g.tiles_m * g.tiles_n;
  if (total > (1 << 30)) return fail(HOT_ERR_UNSUPPORTED, "hot_gemm_i8: too many tiles");
  hipLaunchKernelGGL((gemm_i8_kernel<WM, WN, BITS, OutT>), dim3((unsigned)total), dim3(G_THREADS), lds, st, g);
  return check_launch("gemm_i8_kernel");
}

template <int BITS, typename OutT>
static int pick_tile(GemmArgs& g, hipStream_t st) {
  return launch_gemm<2, 2, BITS, OutT>(g, st);
}

template <int BITS>
static int dispatch_out(int out_dtype, GemmArgs& g, hipStream_t st) {
  switch (out_dtype) {
    case HOT_F32: return pick_tile<BITS, float>(g, st);
    case HOT_BF16: return pick_tile<BITS, bf16_t>(g, st);
    case HOT_F16: return pick_tile<BITS, f16_t>(g, st);
    default: return fail(HOT_ERR_INVALID, "hot_gemm_i8: bad out dtype %d", out_dtype);
  }
}

int gemm_i8_impl(const void* A, int64_t lda, const void* B, int64_t ldb, int bits, int64_t M, int64_t N,
                 int64_t K, const float* scale_a, int a_per_row, const float* scale_b, float post_scale,
                 void* out, int out_dtype, int64_t ldo, int32_t* acc_out, hipStream_t st) {
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
  if (M == 0 || N == 0) return HOT_OK;
  GemmArgs g;
  g.A = (const uint8_t*)A; g.B = (const uint8_t*)B; g.lda = lda; g.ldb = ldb; g.M = M; g.N = N;
  g.ktiles = (int)(kpad / G_BK);
  g.scale_a = scale_a; g.scale_b = scale_b; g.post_scale = post_scale; g.a_per_row = a_per_row;
  g.out = out; g.ldo = ldo; g.acc_out = acc_out;
  return bits == 4 ? dispatch_out<4>(out_dtype, g, st) : dispatch_out<8>(out_dtype, g, st);
}

}  // namespace hot
