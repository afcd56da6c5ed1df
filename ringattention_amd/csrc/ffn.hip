// bf16 MFMA GEMM for gfx950 and the SwiGLU feed-forward built on it: the body that
// blockwise_feedforward (ringattention_jax.py:333-352) scans over chunks of tokens.
//
// GEMM: C (M,N) = op(A) op(B) [+ op(A2) op(B2)], fp32 accumulation in v_mfma_f32_32x32x16_bf16.
//   The tile is chosen per problem: 256 x 256 or 256 x 128 over 4 wavefronts, one per SIMD (gemm_bf16_w4_kernel:
//   each wavefront 128 x 128 or 128 x 64; eight or six operand fragments from LDS per sixteen or eight MFMAs),
//   whichever fills the CUs in fewer weighted rounds; gemm_bf16_kernel with WGM x WGN wavefronts on a BM x BN tile
//   (256 x 128 over 8, 128 x 128 over 4; K step 64, LDS double buffered) for what those do not divide or reach.
//   An operand whose contraction index is contiguous in memory is staged row-major and read with
//   16-byte LDS reads; one whose contraction index is the slow axis is staged as it lies in memory
//   and read with ds_read_b64_tr_b16, so no layout ever needs a transposing copy.
#include "common.hpp"
#include <stdlib.h>

namespace ra {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int GBK = 64;               // K step of the 8-wavefront tiles (and the granularity required of K)

struct GemmArgs {
  const uint16_t* A; const uint16_t* B; const uint16_t* A2; const uint16_t* B2;
  void* C;
  int M, N, K;
  int c_f32, beta_one;
  // two products that share A in one launch, C = A B and C_alt = A B_alt (both (M, N)): the grid covers the tile
  // columns of both, so that the two together fill the CUs in fewer rounds than one after the other (4-wavefront
  // tile kernels only; null: one product)
  const uint16_t* B_alt; void* C_alt;
};

__device__ __forceinline__ s16x4 lds_tr(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p));
}

// Workgroup -> tile.  Workgroups go to the 8 XCDs round-robin and each XCD has its own L2, so XCD x takes the
// contiguous range x of a tile order in which consecutive tiles form groups of GROUP_M tile rows walked column by
// column: the 32 workgroups resident on an XCD then cover about 4 x 8 tiles, an A panel is fetched into that L2
// once per 8 tiles and a B panel once per 4, instead of once per tile.
constexpr int GROUP_M = 4;
__device__ __forceinline__ bool tile_of_block(int ntm, int ntn, int& tm, int& tn) {
  const int ntiles = ntm * ntn;
  const int per_xcd = (ntiles + 7) >> 3;
  const int pid = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (pid >= ntiles) return false;
  const int group = pid / (GROUP_M * ntn), first_m = group * GROUP_M;
  const int rows = min(GROUP_M, ntm - first_m);
  const int in_group = pid - group * GROUP_M * ntn;
  tm = first_m + in_group % rows;
  tn = in_group / rows;
  return true;
}

// One wavefront's accumulators -> C.  A lane holds column lo of each 32 x 32 block, rows 8 (r / 4) + 4 hi + r % 4:
// written straight to memory that is one 4-byte access per lane and register.  Each block goes through a
// 32 x 36 float patch of LDS private to the wavefront instead and leaves as 16 bytes per lane (rows of 128
// bytes).  MODE 0: bf16 C, 1: fp32 C, 2: fp32 C +=.  Blocks alternate between patch0 and patch1 (which may be the
// same): with two patches the LDS writes of a block overlap the reads and stores of the block before.
template <int MODE, int MB, int NB>
__device__ __forceinline__ void store_tile(f32x16 (&acc)[MB][NB], float* patch0, float* patch1, void* C, int ldc,
                                           int row0, int col0, int lane) {
  const int lo = lane & 31, hi = lane >> 5;
  const int er = lane >> 3, ec = (lane & 7) * 4;          // this lane's row (of 8 per pass) and first column
  // MODE 2 adds into C: the old values of a block are requested PF blocks ahead, before the stores of the block in
  // hand.  (Requested inside the block that uses them, every block waited a memory latency and, the counter of
  // outstanding memory operations being in order, for the stores of the block before: sixteen such waits were a third
  // of a workgroup's time at K = 2048.)
  constexpr int PF = 2, NBLK = MB * NB;
  float4 old[PF][4] = {};
#define RA_ST_REQUEST(BI)                                                                               \
  _Pragma("unroll") for (int pass = 0; pass < 4; pass++)                                                \
    old[(BI) % PF][pass] = *(const float4*)((const float*)C + (int64_t)(row0 + ((BI) / NB) * 32 + pass * 8 + er) * ldc + \
                                            col0 + ((BI) % NB) * 32 + ec);
  if (MODE == 2) {
#pragma unroll
    for (int bi = 0; bi < PF && bi < NBLK; bi++) RA_ST_REQUEST(bi)
  }
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int j = 0; j < NB; j++) {
      const int bi = i * NB + j;
      float* patch = (bi & 1) ? patch1 : patch0;
      float4 cur[4] = {};
      if (MODE == 2) {
#pragma unroll
        for (int pass = 0; pass < 4; pass++) cur[pass] = old[bi % PF][pass];
        if (bi + PF < NBLK) RA_ST_REQUEST(bi + PF)
      }
#pragma unroll
      for (int r = 0; r < 16; r++) patch[((r >> 2) * 8 + hi * 4 + (r & 3)) * 36 + lo] = acc[i][j][r];
#pragma unroll
      for (int pass = 0; pass < 4; pass++) {
        const int row = pass * 8 + er;
        const float4 v = *(const float4*)&patch[row * 36 + ec];
        const int64_t o = (int64_t)(row0 + i * 32 + row) * ldc + col0 + j * 32 + ec;
        if (MODE == 0) {
          uint2 w;
          w.x = f32x2_to_bf16x2(v.x, v.y);
          w.y = f32x2_to_bf16x2(v.z, v.w);
          *(uint2*)((uint16_t*)C + o) = w;
        } else {
          float4* c = (float4*)((float*)C + o);
          float4 w = v;
          if (MODE == 2) { w.x += cur[pass].x; w.y += cur[pass].y; w.z += cur[pass].z; w.w += cur[pass].w; }
          *c = w;
        }
      }
    }
#undef RA_ST_REQUEST
}

// TA: A is stored (K,M).  TB: B is stored (N,K).
template <bool TA, bool TB, int BM, int BN, int WGM, int WGN, bool DEEP>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_bf16_kernel(GemmArgs g) {
  constexpr int NT = 64 * WGM * WGN, BK = GBK;
  constexpr int NAT_STR = BK + 8;      // row stride (elements) of a tile read row-wise
  constexpr int WM = BM / WGM, WN = BN / WGN, MB = WM / 32, NB = WN / 32;
  constexpr int A_STR = TA ? BM + 32 : NAT_STR;     // elements
  constexpr int B_STR = TB ? NAT_STR : BN + 32;
  constexpr int A_ROWS = TA ? BK : BM, B_ROWS = TB ? BN : BK;
  constexpr int A_CPR = (TA ? BM : BK) / 8, B_CPR = (TB ? BK : BN) / 8;   // 16-byte chunks per staged row
  constexpr int A_CH = A_ROWS * A_CPR / NT, B_CH = B_ROWS * B_CPR / NT;     // chunks per thread
  static_assert(A_CH * NT == A_ROWS * A_CPR && B_CH * NT == B_ROWS * B_CPR, "tile does not divide over the threads");
  __shared__ __attribute__((aligned(16))) uint16_t As[2][A_ROWS * A_STR];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[2][B_ROWS * B_STR];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int wm = wave / WGN, wn = wave % WGN;
  int tm, tn;
  if (!tile_of_block(g.M / BM, g.N / BN, tm, tn)) return;
  const int m0 = tm * BM, n0 = tn * BN;

  f32x16 acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // staging registers: two sets (P, Q) of named scalars and straight-line code (arrays that stay live
  // across the MFMA section end up in scratch memory).  A K slab is requested two iterations before it
  // is stored to LDS, which covers the global latency under load.
  static_assert(A_CH <= 4 && B_CH <= 4, "at most four 16-byte chunks per thread and operand");
  uint4 Pa0, Pa1, Pa2, Pa3, Pb0, Pb1, Pb2, Pb3, Qa0, Qa1, Qa2, Qa3, Qb0, Qb1, Qb2, Qb3;
  const int lda = TA ? g.M : g.K, ldb = TB ? g.K : g.N;
  const int nk = g.K / BK;
  const int total = nk * (g.A2 ? 2 : 1);
  // chunk c of this thread: staged row and 16-byte column, fixed for the whole kernel
#define RA_A_OFF(C, K0) (TA ? (int64_t)((K0) + ((C) * NT + tid) / A_CPR) * lda + m0 + (((C) * NT + tid) % A_CPR) * 8 \
                            : (int64_t)(m0 + ((C) * NT + tid) / A_CPR) * lda + (K0) + (((C) * NT + tid) % A_CPR) * 8)
#define RA_B_OFF(C, K0) (TB ? (int64_t)(n0 + ((C) * NT + tid) / B_CPR) * ldb + (K0) + (((C) * NT + tid) % B_CPR) * 8 \
                            : (int64_t)((K0) + ((C) * NT + tid) / B_CPR) * ldb + n0 + (((C) * NT + tid) % B_CPR) * 8)
#define RA_A_LDS(C) ((((C) * NT + tid) / A_CPR) * A_STR + (((C) * NT + tid) % A_CPR) * 8)
#define RA_B_LDS(C) ((((C) * NT + tid) / B_CPR) * B_STR + (((C) * NT + tid) % B_CPR) * 8)
  // slab T (clamped to the last one; slabs nk .. 2 nk - 1 belong to the second operand pair)
#define RA_LOAD_STAGE(S, T)                                                                             \
  {                                                                                                     \
    const int t_ = min((T), total - 1);                                                                 \
    const uint16_t* Ap = t_ >= nk ? g.A2 : g.A;                                                         \
    const uint16_t* Bp = t_ >= nk ? g.B2 : g.B;                                                         \
    const int k0_ = (t_ >= nk ? t_ - nk : t_) * BK;                                                    \
    if (A_CH > 0) S##a0 = *(const uint4*)(Ap + RA_A_OFF(0, k0_));                                       \
    if (A_CH > 1) S##a1 = *(const uint4*)(Ap + RA_A_OFF(1, k0_));                                       \
    if (A_CH > 2) S##a2 = *(const uint4*)(Ap + RA_A_OFF(2, k0_));                                       \
    if (A_CH > 3) S##a3 = *(const uint4*)(Ap + RA_A_OFF(3, k0_));                                       \
    if (B_CH > 0) S##b0 = *(const uint4*)(Bp + RA_B_OFF(0, k0_));                                       \
    if (B_CH > 1) S##b1 = *(const uint4*)(Bp + RA_B_OFF(1, k0_));                                       \
    if (B_CH > 2) S##b2 = *(const uint4*)(Bp + RA_B_OFF(2, k0_));                                       \
    if (B_CH > 3) S##b3 = *(const uint4*)(Bp + RA_B_OFF(3, k0_));                                       \
  }
#define RA_STORE_STAGE(S, BUF)                                                                          \
  {                                                                                                     \
    if (A_CH > 0) *(uint4*)(&As[BUF][RA_A_LDS(0)]) = S##a0;                                             \
    if (A_CH > 1) *(uint4*)(&As[BUF][RA_A_LDS(1)]) = S##a1;                                             \
    if (A_CH > 2) *(uint4*)(&As[BUF][RA_A_LDS(2)]) = S##a2;                                             \
    if (A_CH > 3) *(uint4*)(&As[BUF][RA_A_LDS(3)]) = S##a3;                                             \
    if (B_CH > 0) *(uint4*)(&Bs[BUF][RA_B_LDS(0)]) = S##b0;                                             \
    if (B_CH > 1) *(uint4*)(&Bs[BUF][RA_B_LDS(1)]) = S##b1;                                             \
    if (B_CH > 2) *(uint4*)(&Bs[BUF][RA_B_LDS(2)]) = S##b2;                                             \
    if (B_CH > 3) *(uint4*)(&Bs[BUF][RA_B_LDS(3)]) = S##b3;                                             \
  }

  // transpose-read lane offset: 16-lane group reads 4 contraction rows x 16 columns
  const int trA = (8 * hi + ((lane & 15) >> 2)) * A_STR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int trB = (8 * hi + ((lane & 15) >> 2)) * B_STR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

#define RA_COMPUTE(CUR_)                                                                                \
  {                                                                                                     \
    _Pragma("unroll")                                                                                  \
    for (int kk = 0; kk < BK / 16; kk++) {                                                             \
      bf16x8 af[MB], bfr[NB];                                                                           \
    _Pragma("unroll")                                                                                  \
      for (int i = 0; i < MB; i++) {                                                                    \
        if (!TA) {                                                                                      \
          af[i] = *(const bf16x8*)(&As[CUR_][(wm * WM + i * 32 + lo) * A_STR + kk * 16 + hi * 8]);      \
        } else {                                                                                        \
          const uint16_t* p = &As[CUR_][kk * 16 * A_STR + trA + wm * WM + i * 32];                      \
          s16x4 x0 = lds_tr(p), x1 = lds_tr(p + 4 * A_STR);                                             \
          af[i] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));  \
        }                                                                                               \
      }                                                                                                 \
    _Pragma("unroll")                                                                                  \
      for (int j = 0; j < NB; j++) {                                                                    \
        if (TB) {                                                                                       \
          bfr[j] = *(const bf16x8*)(&Bs[CUR_][(wn * WN + j * 32 + lo) * B_STR + kk * 16 + hi * 8]);     \
        } else {                                                                                        \
          const uint16_t* p = &Bs[CUR_][kk * 16 * B_STR + trB + wn * WN + j * 32];                      \
          s16x4 x0 = lds_tr(p), x1 = lds_tr(p + 4 * B_STR);                                             \
          bfr[j] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7)); \
        }                                                                                               \
      }                                                                                                 \
    _Pragma("unroll")                                                                                  \
      for (int i = 0; i < MB; i++)                                                                      \
    _Pragma("unroll")                                                                                  \
        for (int j = 0; j < NB; j++)                                                                    \
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);       \
    }                                                                                                   \
  }
  RA_LOAD_STAGE(P, 0);
  RA_STORE_STAGE(P, 0);
  if (DEEP) {
    RA_LOAD_STAGE(Q, 1);
    RA_LOAD_STAGE(P, 2);
    __syncthreads();
    for (int it = 0; it < total; it += 2) {
      // slab it is in buffer 0; slab it + 1 goes to buffer 1, slab it + 3 is requested
      RA_STORE_STAGE(Q, 1);
      RA_LOAD_STAGE(Q, it + 3);
      __builtin_amdgcn_sched_barrier(0);
      RA_COMPUTE(0);
      __syncthreads();
      if (it + 1 >= total) break;
      RA_STORE_STAGE(P, 0);
      RA_LOAD_STAGE(P, it + 4);
      __builtin_amdgcn_sched_barrier(0);
      RA_COMPUTE(1);
      __syncthreads();
    }
  } else {
    // one register set (the tile's accumulators leave no room for two): a slab is in flight for one iteration
    __syncthreads();
    for (int it = 0; it < total; it++) {
      const int cur = it & 1;
      RA_LOAD_STAGE(P, it + 1);
      __builtin_amdgcn_sched_barrier(0);
      RA_COMPUTE(cur);
      RA_STORE_STAGE(P, cur ^ 1);
      __syncthreads();
    }
  }
#undef RA_COMPUTE
#undef RA_LOAD_STAGE
#undef RA_STORE_STAGE
#undef RA_A_OFF
#undef RA_B_OFF
#undef RA_A_LDS
#undef RA_B_LDS

  // epilogue through one LDS patch per wavefront (the operand tiles are dead by now)
  __syncthreads();
  static_assert(sizeof(As) >= (size_t)NT / 64 * 32 * 36 * sizeof(float), "operand tile too small for the epilogue patches");
  float* patch = (float*)&As[0][0] + wave * (32 * 36);
  if (!g.c_f32) store_tile<0>(acc, patch, patch, g.C, g.N, m0 + wm * WM, n0 + wn * WN, lane);
  else if (!g.beta_one) store_tile<1>(acc, patch, patch, g.C, g.N, m0 + wm * WM, n0 + wn * WN, lane);
  else store_tile<2>(acc, patch, patch, g.C, g.N, m0 + wm * WM, n0 + wn * WN, lane);
}

// 256 x BN tile (BN 256 or 128) over FOUR wavefronts (2 x 2), one per SIMD with all 512 registers: each wavefront
// owns 128 x BN/2 of C (256 accumulator registers at BN = 256), so a K slice of 16 takes eight operand fragments from
// LDS for sixteen MFMAs - half the LDS bytes per MFMA of the eight-wavefront tile.  With a single wavefront per SIMD
// nothing hides latency but the wavefront's own pipelining, and what the loop costs beside its MFMAs is mostly the
// energy of moving operands (the board runs it at its power limit), so:
//   * operands go from global memory straight into LDS (buffer_load ... lds: sixteen bytes a lane, the 64 lanes of
//     an instruction fill 1 KB of consecutive LDS): no staging registers, no LDS writes by the wavefronts;
//   * the unit is a slab of 64 K positions (four K slices) of the whole tile, 32 KB an operand at BN = 256, fetched
//     as whole 128-byte lines whichever way the operand lies;
//   * A has three slab buffers and B two (160 KB at BN = 256), so that a slab step can issue its loads evenly - B's
//     in its first and last quarter, A's in the second and third, four a wavefront and quarter - and every load has
//     between 2.5 quarters and a whole slab step to land;
//   * the barrier between slabs is a bare s_barrier behind an s_waitcnt that leaves the eight newest loads (the slab
//     after next of A) in flight; __syncthreads() would wait for all of them.
// LDS layout of a slab.  Row-wise operand (rows run along K: A unless TA, B if TB): one row of 64 elements = eight
// 16-byte chunks per tile row, chunk c of row r at position c ^ ((r >> 1) & 7).  K-major operand (stored (K, M) or
// (K, N)): 64 rows of W = 256 or BN elements, chunk c of row r at position c ^ ((r & 3) << 2).  Both make the
// fragment reads (16-byte reads of a row-wise slab, ds_read_b64_tr_b16 of a K-major one) conflict-free without
// padding, and the permutation is done by the loads: lane l of a load fetches the chunk that belongs at position l.
template <bool TA, bool TB, int BN>
__global__ __launch_bounds__(256) void gemm_bf16_w4_kernel(GemmArgs g) {
  static_assert(BN == 256 || BN == 128, "tile width");
  // NJ: 32-column blocks of a wavefront's part of C; NBC: loads per wavefront for half a slab of B
  constexpr int BM = 256, WM = 128, WN = BN / 2, NJ = WN / 32, NBC = BN / 64, SK = 64, WS = 64;
  __shared__ __attribute__((aligned(16))) uint16_t As0[BM * SK];
  __shared__ __attribute__((aligned(16))) uint16_t As1[BM * SK];
  __shared__ __attribute__((aligned(16))) uint16_t As2[BM * SK];
  __shared__ __attribute__((aligned(16))) uint16_t Bs0[BN * SK];
  __shared__ __attribute__((aligned(16))) uint16_t Bs1[BN * SK];
#define RA_W4_AS(BUF) ((BUF) == 0 ? As0 : (BUF) == 1 ? As1 : As2)
#define RA_W4_BS(BUF) ((BUF) ? Bs1 : Bs0)

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  const int ntn1 = g.N / BN;
  if (!tile_of_block(g.M / BM, g.B_alt ? 2 * ntn1 : ntn1, tm, tn)) return;
  if (tn >= ntn1) { tn -= ntn1; g.B = g.B_alt; g.C = g.C_alt; }       // a tile of the second product
  const int m0 = tm * BM, n0 = tn * BN;

  f32x16 acc[4][NJ];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int lda = TA ? g.M : g.K, ldb = TB ? g.K : g.N;
  const int nk = g.K / SK;                         // slabs per operand pair
  const int nslab = nk * (g.A2 ? 2 : 1);
  // Load c of a wavefront for half a slab.  Row-wise: rows (4 c + wave) 8 .. + 7 of the half's 128 (BN / 2) tile
  // rows, lane l row l / 8, position l % 8.  K-major: the half's 32 K rows, RPI = 64 / (W / 8) rows an instruction,
  // lane l row l / (W / 8), position l % (W / 8).  The lane offset (bytes) is the same for every c but for the rows.
  constexpr int A_CPR = TA ? BM / 8 : 8, B_CPR = TB ? 8 : BN / 8;         // chunks per LDS row
  constexpr int A_RPI = 64 / A_CPR, B_RPI = 64 / B_CPR;                   // rows per load instruction
  const int ar = lane / A_CPR, br = lane / B_CPR;
  const int a_sw = TA ? ((wave * A_RPI + ar) & 3) << 2 : (((wave * 8 + ar) >> 1) & 7);
  const int b_sw = TB ? (((wave * 8 + br) >> 1) & 7) : ((wave * B_RPI + br) & 3) << 2;
  const uint32_t ga0 = 2u * (uint32_t)((wave * A_RPI + ar) * lda + ((lane % A_CPR) ^ a_sw) * 8);
  const uint32_t gb0 = 2u * (uint32_t)((wave * B_RPI + br) * ldb + ((lane % B_CPR) ^ b_sw) * 8);
  const uint32_t ga_c = 2u * (uint32_t)(4 * A_RPI * lda), gb_c = 2u * (uint32_t)(4 * B_RPI * ldb);   // per c
  // A slab is read through a buffer descriptor at its own origin in the tile (64-bit scalar arithmetic), so the 32-bit
  // lane and scalar offsets only span one slab - at most 256 rows of a row-wise operand, 64 of a K-major one - and
  // an operand may be of any size.  Elements from one slab to the next, and bytes to a slab's second half:
  const int64_t a_slab = TA ? (int64_t)lda * SK : SK, b_slab = TB ? SK : (int64_t)ldb * SK;
  const uint32_t a_half = TA ? 2u * (uint32_t)lda * 32 : 2u * (uint32_t)lda * 128;
  const uint32_t b_half = TB ? 2u * (uint32_t)ldb * (BN / 2) : 2u * (uint32_t)ldb * 32;
  const int64_t tile_a = TA ? (int64_t)m0 : (int64_t)m0 * lda, tile_b = TB ? (int64_t)n0 * ldb : (int64_t)n0;
  const uint16_t* const a_tile = g.A + tile_a;
  const uint16_t* const b_tile = g.B + tile_b;
  const uint16_t* const a2_tile = (g.A2 ? g.A2 : g.A) + tile_a;
  const uint16_t* const b2_tile = (g.B2 ? g.B2 : g.B) + tile_b;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  // half HF of slab J into buffer BUF (J past the end: the last slab again, into a buffer nobody reads any more)
#define RA_W4_LOAD_A(BUF, J, HF)                                                                        \
  {                                                                                                     \
    const int j_ = min((J), nslab - 1);                                                                 \
    const bool second_ = j_ >= nk;                                                                      \
    const __amdgpu_buffer_rsrc_t r_ = __builtin_amdgcn_make_buffer_rsrc(                               \
        (void*)((second_ ? a2_tile : a_tile) + (second_ ? j_ - nk : j_) * a_slab), 0, 0x7fffffff, 0x00020000); \
    const uint32_t so_ = (HF) * a_half;                                                                 \
    _Pragma("unroll") for (int c = 0; c < 4; c++)                                                       \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                         \
          r_, (lds_ptr)&RA_W4_AS(BUF)[(HF) * (BM * SK / 2) + (4 * c + wave) * 512], 16, ga0 + c * ga_c, so_, 0, 0); \
  }
#define RA_W4_LOAD_B(BUF, J, HF)                                                                        \
  {                                                                                                     \
    const int j_ = min((J), nslab - 1);                                                                 \
    const bool second_ = j_ >= nk;                                                                      \
    const __amdgpu_buffer_rsrc_t r_ = __builtin_amdgcn_make_buffer_rsrc(                               \
        (void*)((second_ ? b2_tile : b_tile) + (second_ ? j_ - nk : j_) * b_slab), 0, 0x7fffffff, 0x00020000); \
    const uint32_t so_ = (HF) * b_half;                                                                 \
    _Pragma("unroll") for (int c = 0; c < NBC; c++)                                                     \
      __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                         \
          r_, (lds_ptr)&RA_W4_BS(BUF)[(HF) * (BN * SK / 2) + (4 * c + wave) * 512], 16, gb0 + c * gb_c, so_, 0, 0); \
  }
  // fragment addresses (elements).  Row-wise, K slice q: row lo, chunk (2 q + hi) ^ ((lo >> 1) & 7): q only flips
  // bits 4 and 5.  K-major, block i: rows 16 q + 8 hi + r4 (and + 4), r4 = (lane & 15) >> 2, columns 32 i + 16 x + 4 y:
  // block b = 32 i / 32 + (the wavefront's first block) of the row, chunk 4 b + 2 x + y / 2 at position
  // ((b ^ r4) << 2) + 2 x + y / 2: one address per block.
  const int r4 = (lane & 15) >> 2, cl = 2 * ((lane >> 4) & 1) + ((lane >> 1) & 1);
  const int natA = (wm * WM + lo) * WS + (hi ^ ((lo >> 1) & 7)) * 8, natB = (wn * WN + lo) * WS + (hi ^ ((lo >> 1) & 7)) * 8;
  const int trA_ = (8 * hi + r4) * BM + cl * 8 + 4 * (lane & 1), trB_ = (8 * hi + r4) * BN + cl * 8 + 4 * (lane & 1);
  const int ba = wm * 4, bb = wn * NJ;             // first 32-column block of this wavefront in a row of the slab
  const int trA0 = trA_ + (((ba + 0) ^ r4) << 5), trA1 = trA_ + (((ba + 1) ^ r4) << 5);
  const int trA2 = trA_ + (((ba + 2) ^ r4) << 5), trA3 = trA_ + (((ba + 3) ^ r4) << 5);
  const int trB0 = trB_ + (((bb + 0) ^ r4) << 5), trB1 = trB_ + (((bb + 1) ^ r4) << 5);
  const int trB2 = trB_ + (((bb + 2) ^ r4) << 5), trB3 = trB_ + (((bb + 3) ^ r4) << 5);
#define RA_W4_SEL(X, I) ((I) == 0 ? X##0 : (I) == 1 ? X##1 : (I) == 2 ? X##2 : X##3)
  // the fragments of K slice Q (0-3) of the slabs in buffers ABUF, BBUF into set F (F##a[0..3], F##b[0..NJ-1])
#define RA_W4_FRAGS(F, ABUF, BBUF, Q)                                                                   \
  _Pragma("unroll") for (int i = 0; i < 4; i++) {                                                       \
    if (!TA) {                                                                                          \
      F##a[i] = *(const bf16x8*)(&RA_W4_AS(ABUF)[(natA ^ ((Q) << 4)) + i * 32 * WS]);                   \
    } else {                                                                                            \
      const uint16_t* p = &RA_W4_AS(ABUF)[RA_W4_SEL(trA, i) + (Q) * 16 * BM];                           \
      s16x4 x0 = lds_tr(p), x1 = lds_tr(p + 4 * BM);                                                    \
      F##a[i] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));    \
    }                                                                                                   \
    if (i >= NJ) continue;                                                                              \
    if (TB) {                                                                                           \
      F##b[i] = *(const bf16x8*)(&RA_W4_BS(BBUF)[(natB ^ ((Q) << 4)) + i * 32 * WS]);                   \
    } else {                                                                                            \
      const uint16_t* p = &RA_W4_BS(BBUF)[RA_W4_SEL(trB, i) + (Q) * 16 * BN];                           \
      s16x4 x0 = lds_tr(p), x1 = lds_tr(p + 4 * BN);                                                    \
      F##b[i] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));    \
    }                                                                                                   \
  }
#define RA_W4_MFMA(F)                                                                                   \
  _Pragma("unroll") for (int i = 0; i < 4; i++)                                                         \
    _Pragma("unroll") for (int j = 0; j < NJ; j++)                                                      \
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F##a[i], F##b[j], acc[i][j], 0, 0, 0);
  // A single wavefront per SIMD issues in order: the MFMA pipe only stays busy if every MFMA is followed by at most
  // a few other instructions.  One group per MFMA of a quarter: the MFMA, its share of the quarter's LDS reads, and
  // every (NM / LOADS)-th a load.
  constexpr int NM = 4 * NJ, RD = (TA ? 8 : 4) + (TB ? NJ : 2 * NJ), RPG = (RD + NM - 1) / NM;
#define RA_W4_SCHED(LOADS)                                                                              \
  _Pragma("unroll") for (int m_ = 0; m_ < NM; m_++) {                                                   \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                  \
    if (m_ * RPG < RD) __builtin_amdgcn_sched_group_barrier(0x100, RPG, 0);                             \
    if (m_ % (NM / (LOADS)) == 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                    \
  }
  // slab J: A in buffer AC (of three), B in buffer BC (of two); its slice 0 already in set F
#define RA_W4_STEP(AC, BC, J)                                                                           \
  {                                                                                                     \
    RA_W4_FRAGS(G, AC, BC, 1);                                                                          \
    RA_W4_LOAD_B((BC) ^ 1, (J) + 1, 1);                                                                 \
    RA_W4_MFMA(F);                                                                                      \
    RA_W4_SCHED(NBC);                                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_W4_FRAGS(F, AC, BC, 2);                                                                          \
    RA_W4_LOAD_A(((AC) + 2) % 3, (J) + 2, 0);                                                           \
    RA_W4_MFMA(G);                                                                                      \
    RA_W4_SCHED(4);                                                                                     \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_W4_FRAGS(G, AC, BC, 3);                                                                          \
    RA_W4_LOAD_A(((AC) + 2) % 3, (J) + 2, 1);                                                           \
    RA_W4_MFMA(F);                                                                                      \
    RA_W4_SCHED(4);                                                                                     \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    /* everything but the slab after next of A (the eight newest loads) has landed, in every wavefront */ \
    asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");                            \
    RA_W4_FRAGS(F, ((AC) + 1) % 3, (BC) ^ 1, 0);                                                        \
    RA_W4_LOAD_B(BC, (J) + 2, 0);                                                                       \
    RA_W4_MFMA(G);                                                                                      \
    RA_W4_SCHED(NBC);                                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
  }
  bf16x8 Fa[4], Fb[NJ], Ga[4], Gb[NJ];
  RA_W4_LOAD_A(0, 0, 0); RA_W4_LOAD_A(0, 0, 1);
  RA_W4_LOAD_B(0, 0, 0); RA_W4_LOAD_B(0, 0, 1);
  RA_W4_LOAD_A(1, 1, 0); RA_W4_LOAD_A(1, 1, 1);
  RA_W4_LOAD_B(1, 1, 0);
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  RA_W4_FRAGS(F, 0, 0, 0);
  // the buffers come round every six slabs
  int j = 0;
  for (; j + 6 <= nslab; j += 6) {
    RA_W4_STEP(0, 0, j);
    RA_W4_STEP(1, 1, j + 1);
    RA_W4_STEP(2, 0, j + 2);
    RA_W4_STEP(0, 1, j + 3);
    RA_W4_STEP(1, 0, j + 4);
    RA_W4_STEP(2, 1, j + 5);
  }
  if (j < nslab) RA_W4_STEP(0, 0, j);
  if (j + 1 < nslab) RA_W4_STEP(1, 1, j + 1);
  if (j + 2 < nslab) RA_W4_STEP(2, 0, j + 2);
  if (j + 3 < nslab) RA_W4_STEP(0, 1, j + 3);
  if (j + 4 < nslab) RA_W4_STEP(1, 0, j + 4);
#undef RA_W4_STEP
#undef RA_W4_AS
#undef RA_W4_BS
#undef RA_W4_SEL
#undef RA_W4_MFMA
#undef RA_W4_FRAGS
#undef RA_W4_LOAD_A
#undef RA_W4_LOAD_B
#undef RA_W4_SCHED

  // epilogue through two LDS patches per wavefront (the operand slabs are dead by now, and no load may land in
  // them any more)
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  static_assert(sizeof(As0) >= (size_t)2 * 32 * 36 * sizeof(float) && sizeof(Bs0) >= (size_t)2 * 32 * 36 * sizeof(float),
                "operand tile too small for two epilogue patches");
  float* patch = (float*)(wave == 0 ? &As0[0] : wave == 1 ? &As1[0] : wave == 2 ? &Bs0[0] : &Bs1[0]);
  if (!g.c_f32) store_tile<0>(acc, patch, patch + 32 * 36, g.C, g.N, m0 + wm * WM, n0 + wn * WN, lane);
  else if (!g.beta_one) store_tile<1>(acc, patch, patch + 32 * 36, g.C, g.N, m0 + wm * WM, n0 + wn * WN, lane);
  else store_tile<2>(acc, patch, patch + 32 * 36, g.C, g.N, m0 + wm * WM, n0 + wn * WN, lane);
}
template <bool TA, bool TB, int BN>
static int launch_w4(const GemmArgs& g, hipStream_t s) {
  const long long nwg = ((long long)(g.M / 256) * (g.N / BN) * (g.B_alt ? 2 : 1) + 7) / 8 * 8;
  gemm_bf16_w4_kernel<TA, TB, BN><<<dim3((unsigned)nwg), 256, 0, s>>>(g);
  RA_CHECK_LAUNCH("gemm_bf16_w4");
  return RA_OK;
}

template <bool TA, bool TB, int BM, int BN, int WGM, int WGN, bool DEEP>
static int launch_tile(const GemmArgs& g, hipStream_t s) {
  const long long nwg = ((long long)(g.M / BM) * (g.N / BN) + 7) / 8 * 8;    // whole rounds over the 8 XCDs
  gemm_bf16_kernel<TA, TB, BM, BN, WGM, WGN, DEEP><<<dim3((unsigned)nwg), 64 * WGM * WGN, 0, s>>>(g);
  RA_CHECK_LAUNCH("gemm_bf16");
  return RA_OK;
}

// Tile choice.  One workgroup of the large tiles fills a CU, so the grid runs in rounds of (number of CUs)
// workgroups: take the tile whose rounds, weighted by what a round of it costs (measured on full grids: a round of
// 256 x 256 tiles takes 1.72 times one of 256 x 128 over four wavefronts, which does half the work), take least.
static bool w4_reach_ok(int M, int N, int K) {
  // the 4-wavefront kernels address a slab through a buffer descriptor at its origin with 32-bit byte offsets: 256
  // rows of a row-wise operand (512 K bytes) or 64 rows of a K-major one (128 M or 128 N bytes) must stay below 2^31
  return M % 256 == 0 && K < (1 << 21) && M < (1 << 23) && N < (1 << 23);
}
static int pick_tile(int M, int N, int K) {
  static const int ncu = [] {     // initialised once, thread-safe
    int dev = 0, n = 0;
    hipDeviceProp_t pr;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&pr, dev) == hipSuccess) n = pr.multiProcessorCount;
    return n > 0 ? n : 256;
  }();
  auto rounds = [&](int bm, int bn) { return ceil((double)(M / bm) * (N / bn) / ncu); };
  const bool w4 = w4_reach_ok(M, N, K);
  int best = 2;
  double cost = rounds(128, 128) * 0.70;
  if (M % 256 == 0 && rounds(256, 128) * 1.16 < cost) { best = 1; cost = rounds(256, 128) * 1.16; }
  if (w4 && rounds(256, 128) * 1.00 < cost) { best = 3; cost = rounds(256, 128) * 1.00; }
  if (w4 && N % 256 == 0 && rounds(256, 256) * 1.72 <= cost) { best = 0; cost = rounds(256, 256) * 1.72; }
  return best;
}

// tile: -1 = pick_tile, else the tile kernel to force (0: 256 x 256 over four wavefronts, 1: 256 x 128 over eight,
// 2: 128 x 128, 3: 256 x 128 over four), which still falls back to another one when the shape does not divide
template <bool TA, bool TB>
static int launch_gemm(const GemmArgs& g, int tile, hipStream_t s) {
  if (g.M % 128 || g.N % 128 || g.K % GBK) {
    set_error("gemm_bf16: M, N must be multiples of 128 and K of 64 (got %d, %d, %d)", g.M, g.N, g.K);
    return RA_ERR_UNSUPPORTED;
  }
  int t = tile >= 0 ? tile : pick_tile(g.M, g.N, g.K);
  if (t == 0 && g.N % 256) t = 3;
  if ((t == 0 || t == 3) && !w4_reach_ok(g.M, g.N, g.K)) t = 1;
  if (t == 1 && g.M % 256) t = 2;
  switch (t) {
    case 0: return launch_w4<TA, TB, 256>(g, s);
    case 3: return launch_w4<TA, TB, 128>(g, s);
    case 1: return launch_tile<TA, TB, 256, 128, 4, 2, true>(g, s);
    default: return launch_tile<TA, TB, 128, 128, 2, 2, false>(g, s);
  }
}

static int gemm_dispatch(const GemmArgs& g, int ta, int tb, int tile, hipStream_t s) {
  if (ta && tb) return launch_gemm<true, true>(g, tile, s);
  if (ta) return launch_gemm<true, false>(g, tile, s);
  if (tb) return launch_gemm<false, true>(g, tile, s);
  return launch_gemm<false, false>(g, tile, s);
}

int gemm_bf16(const void* A, const void* B, void* C, int M, int N, int K, int ta, int tb, int c_dtype, int beta_one,
              int tile, hipStream_t s) {
  GemmArgs g{(const uint16_t*)A, (const uint16_t*)B, nullptr, nullptr, C, M, N, K, c_dtype == RA_F32, beta_one};
  return gemm_dispatch(g, ta, tb, tile, s);
}

// C1 = A B1 and C2 = A B2 (both (M, N), row-major, bf16 out), in one launch where the 4-wavefront tile kernels take
// the shape, else one after the other.  Same bits either way: a tile is computed the same whichever launch holds it.
int gemm_bf16_pair(const void* A, const void* B1, const void* B2, void* C1, void* C2, int M, int N, int K,
                          int tile, hipStream_t s) {
  if (M % 256 == 0 && N % 128 == 0 && K % GBK == 0 && w4_reach_ok(M, N, K)) {
    int t = tile >= 0 ? tile : pick_tile(M, 2 * N, K);
    if (t == 0 && N % 256) t = 3;
    if (t == 0 || t == 3) {
      GemmArgs g{(const uint16_t*)A, (const uint16_t*)B1, nullptr, nullptr, C1, M, N, K, 0, 0, (const uint16_t*)B2, C2};
      return t == 0 ? launch_w4<false, false, 256>(g, s) : launch_w4<false, false, 128>(g, s);
    }
  }
  if (int rc = gemm_bf16(A, B1, C1, M, N, K, 0, 0, RA_BF16, 0, tile, s)) return rc;
  return gemm_bf16(A, B2, C2, M, N, K, 0, 0, RA_BF16, 0, tile, s);
}

// ------------------------------------------------------------------ SwiGLU elementwise parts
__device__ __forceinline__ float silu(float x) { return x / (1.f + __expf(-x)); }

__global__ void swiglu_act_kernel(const uint16_t* a, const uint16_t* b, uint16_t* h, int64_t n8) {
  // 8 elements (16 bytes) per thread
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
    uint4 ua = ((const uint4*)a)[i], ub = ((const uint4*)b)[i], uh;
    const uint16_t* pa = (const uint16_t*)&ua; const uint16_t* pb = (const uint16_t*)&ub; uint16_t* ph = (uint16_t*)&uh;
#pragma unroll
    for (int e = 0; e < 8; e++) ph[e] = f32_to_bf16(silu(bf16_to_f32(pa[e])) * bf16_to_f32(pb[e]));
    ((uint4*)h)[i] = uh;
  }
}

__global__ void swiglu_act_bwd_kernel(const uint16_t* a, const uint16_t* b, const uint16_t* dh, uint16_t* h,
                                      uint16_t* da, uint16_t* db, int64_t n8) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
    uint4 ua = ((const uint4*)a)[i], ub = ((const uint4*)b)[i], ud = ((const uint4*)dh)[i], uh, uda, udb;
    const uint16_t* pa = (const uint16_t*)&ua; const uint16_t* pb = (const uint16_t*)&ub;
    const uint16_t* pd = (const uint16_t*)&ud;
    uint16_t* ph = (uint16_t*)&uh; uint16_t* pda = (uint16_t*)&uda; uint16_t* pdb = (uint16_t*)&udb;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float av = bf16_to_f32(pa[e]), bv = bf16_to_f32(pb[e]), dv = bf16_to_f32(pd[e]);
      const float sg = 1.f / (1.f + __expf(-av));
      const float sl = av * sg;
      ph[e] = f32_to_bf16(sl * bv);
      pdb[e] = f32_to_bf16(dv * sl);
      pda[e] = f32_to_bf16(dv * bv * (sg * (1.f + av * (1.f - sg))));   // d silu / da
    }
    ((uint4*)h)[i] = uh; ((uint4*)da)[i] = uda; ((uint4*)db)[i] = udb;
  }
}

static int check_ffn_shape(const ra_swiglu_params* p, const char* who) {
  if (p->T % 128 || p->d % 128 || p->f % 128) {
    set_error("%s: tokens, hidden and intermediate sizes must be multiples of 128 (got %d, %d, %d)", who, p->T,
              p->d, p->f);
    return RA_ERR_UNSUPPORTED;
  }
  return RA_OK;
}

int swiglu_fwd(const ra_swiglu_params* p, hipStream_t s) {
  if (int rc = check_ffn_shape(p, "swiglu_fwd")) return rc;
  const int T = p->T, d = p->d, f = p->f, tile = p->gemm_tile - 1;
  if (int rc = gemm_bf16_pair(p->x, p->w1, p->w3, p->a, p->b, T, f, d, tile, s)) return rc;     // a = x w1, b = x w3
  const int64_t n8 = (int64_t)T * f / 8;
  swiglu_act_kernel<<<2048, 256, 0, s>>>((const uint16_t*)p->a, (const uint16_t*)p->b, (uint16_t*)p->h, n8);
  RA_CHECK_LAUNCH("swiglu_act");
  return gemm_bf16(p->h, p->w2, p->y, T, d, f, 0, 0, RA_BF16, 0, tile, s);                 // y = h w2
}

int swiglu_weight_grads(const ra_swiglu_params* p, hipStream_t s) {
  if (int rc = check_ffn_shape(p, "swiglu_weight_grads")) return rc;
  const int T = p->T, d = p->d, f = p->f, tile = p->gemm_tile - 1;
  if (int rc = gemm_bf16(p->x, p->da, p->dw1, d, f, T, 1, 0, RA_F32, 1, tile, s)) return rc;
  if (int rc = gemm_bf16(p->x, p->db, p->dw3, d, f, T, 1, 0, RA_F32, 1, tile, s)) return rc;
  return gemm_bf16(p->h, p->dy, p->dw2, f, d, T, 1, 0, RA_F32, 1, tile, s);
}

int swiglu_bwd(const ra_swiglu_params* p, hipStream_t s) {
  if (int rc = check_ffn_shape(p, "swiglu_bwd")) return rc;
  const int T = p->T, d = p->d, f = p->f, tile = p->gemm_tile - 1;
  // recompute the pre-activations (nothing_saveable) unless the caller kept them, then
  //   dh = dy w2^T ; da, db from the activation ; dx = da w1^T + db w3^T
  //   dw1 += x^T da ; dw3 += x^T db ; dw2 += h^T dy
  if (!p->preact_saved) {
    if (int rc = gemm_bf16_pair(p->x, p->w1, p->w3, p->a, p->b, T, f, d, tile, s)) return rc;
  }
  // dh goes into the da buffer first, the activation backward then rewrites it in place
  if (int rc = gemm_bf16(p->dy, p->w2, p->da, T, f, d, 0, 1, RA_BF16, 0, tile, s)) return rc;
  const int64_t n8 = (int64_t)T * f / 8;
  swiglu_act_bwd_kernel<<<2048, 256, 0, s>>>((const uint16_t*)p->a, (const uint16_t*)p->b, (const uint16_t*)p->da,
                                             (uint16_t*)p->h, (uint16_t*)p->da, (uint16_t*)p->db, n8);
  RA_CHECK_LAUNCH("swiglu_act_bwd");
  GemmArgs g{(const uint16_t*)p->da, (const uint16_t*)p->w1, (const uint16_t*)p->db, (const uint16_t*)p->w3,
             p->dx, T, d, f, 0, 0};
  if (int rc = gemm_dispatch(g, 0, 1, tile, s)) return rc;                                  // dx
  return p->defer_weight_grads ? RA_OK : swiglu_weight_grads(p, s);
}

}  // namespace ra
