// bfloat16 matrix products on the matrix cores (MFMA), 32-bit accumulation, fused epilogue:
//   y = act(a . w^T + bias) (+ residual),  a [M, K] (row stride lda), w [N, K], y [M, N] bf16 or f32.
// Three kernels, chosen by M:
//   tile kernel   (M > 128): a 256x256, 256x192, 256x128, 128x128 or 128x64 tile per workgroup of 4 waves, 32x32x16 MFMA,
//                 (K split into ranges, with a second kernel for the sums, where the tiles alone would leave CUs idle)
//                 operands staged through LDS (two buffers), the next k-tile's global loads in registers meanwhile;
//   stream kernel (M <= 128; up to 24 rows where an estimate puts it ahead of the skinny kernel: long sums, workgroup counts
//                 that do not fit the CUs): the weights are the traffic; `a` is shared through LDS by the 4 to 16 waves of a
//                 workgroup, the weights go straight into MFMA operand registers, K is split over workgroups
//                 and a second kernel adds the partial sums in a fixed order;
//   skinny kernel (M <= 24, and up to 64 rows of narrow layers, see use_skinny): a workgroup owns 16 output columns;
//                 its waves split K, load their part of w
//                 straight into MFMA operand registers (16x16x32), and their partial sums are added
//                 through LDS in a fixed order.
// No atomics anywhere: results are deterministic. K and lda must be multiples of 8 (16-byte operand loads);
// any M and N.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}

__device__ __forceinline__ u32x4 load16(const bf16_t* p) { return *reinterpret_cast<const u32x4*>(p); }

template <typename TO>
__device__ __forceinline__ void epilogue_store(float v, int m, int n, const float* bias, const float* residual, long ldr,
                                               TO* out, long ldo, int act) {
  if (bias) v += bias[n];
  v = lev_activate(v, act);
  if (residual) v += residual[(size_t)m * ldr + n];
  out[(size_t)m * ldo + n] = from_float<TO>(v);
}

// ------------------------------------------------------------------------------------------------
// Tile kernel. A workgroup of 4 waves (2 x 2) computes a BM x BN tile; a wave computes (BM/2) x (BN/2)
// with 32x32x16 MFMA. The larger the wave's tile, the fewer LDS bytes per MFMA: 64 x 64 per wave needs
// the whole LDS bandwidth, 128 x 128 half of it. Operand tiles of BK = 64 go global -> registers -> LDS
// (two LDS buffers, one barrier per k-tile). With one wave per SIMD nothing else fills the matrix pipe
// while a wave issues loads and LDS traffic, so those are interleaved one by one between the products.
// Workgroups are numbered so that each XCD (id % 8) works on a contiguous band of tiles and shares
// operands in its own L2.
#define TK 64
#define LDS_STRIDE 72  // bf16 elements per LDS row: 64 + 8 of padding (144 bytes): 16-byte reads without bank conflicts

template <typename TO>
__device__ __forceinline__ void store_vec4(TO* p, const float v[4]);
template <>
__device__ __forceinline__ void store_vec4<float>(float* p, const float v[4]) {
  *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
}
template <>
__device__ __forceinline__ void store_vec4<bf16_t>(bf16_t* p, const float v[4]) {
  typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
  *reinterpret_cast<u32x2*>(p) = u32x2{float2_to_bf16x2(v[0], v[1]), float2_to_bf16x2(v[2], v[3])};
}

// Output of a wave's (TI x 32) x (TJ x 32) accumulators through an LDS area of its own: 32 rows at a time are
// staged and written out as rows of 4 consecutive columns per lane, so that stores are wide and coalesced.
// No barrier: LDS executes a wave's instructions in order, and a barrier that also waited for the global
// stores (as __syncthreads() does) would expose their latency once per 32 rows.
// 32x32 accumulator: register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32.
template <typename TO, int ACT, int TI, int TJ>
__device__ __forceinline__ void tile_epilogue(const f32x16 (&acc)[TI][TJ], float* Cs, int lane, int mw, int nw,
                                              const float* __restrict__ bias, const float* residual, long ldr, TO* out,
                                              long ldo, int M, int N, int act, int vec_ok) {
  constexpr int WN = TJ * 32, CS = WN + 4;
  constexpr int QUADS = WN / 4;           // groups of 4 columns in a staged row
  constexpr int TURNS = 32 * QUADS / 64;  // per lane and 32 rows
  constexpr int UNROLL_TURNS = ACT >= 0 ? 4 : 1;
#pragma unroll
  for (int i = 0; i < TI; ++i) {
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) Cs[((r >> 2) * 8 + (lane >> 5) * 4 + (r & 3)) * CS + j * 32 + (lane & 31)] = acc[i][j][r];
#pragma unroll UNROLL_TURNS
    for (int q = 0; q < TURNS; ++q) {  // four LDS reads in flight where the activation's code is short
      const int idx = lane + 64 * q;
      const int row = idx / QUADS, c4 = idx % QUADS;
      const int m = mw + i * 32 + row;
      const int n = nw + c4 * 4;
      const f32x4 cv = *reinterpret_cast<const f32x4*>(&Cs[row * CS + c4 * 4]);
      if (m >= M || n >= N) continue;
      float v[4] = {cv[0], cv[1], cv[2], cv[3]};
      const bool whole = vec_ok && n + 3 < N;
      if (bias) {
        if (whole) {
          const f32x4 b = *reinterpret_cast<const f32x4*>(bias + n);
          v[0] += b[0]; v[1] += b[1]; v[2] += b[2]; v[3] += b[3];
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += bias[min(n + e, N - 1)];
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)  // the exact GELU of a bfloat16 output takes the short erf
        v[e] = (ACT == LEV_ACT_GELU_ERF && sizeof(TO) == 2) ? lev_gelu_erf_coarse(v[e]) : lev_activate_as<ACT>(v[e], act);
      if (residual) {
        const float* rrow = residual + (size_t)m * ldr;
        if (whole) {
          const f32x4 rr = *reinterpret_cast<const f32x4*>(rrow + n);
          v[0] += rr[0]; v[1] += rr[1]; v[2] += rr[2]; v[3] += rr[3];
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += rrow[min(n + e, N - 1)];
        }
      }
      TO* orow = out + (size_t)m * ldo + n;
      if (whole) {
        store_vec4<TO>(orow, v);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) orow[e] = from_float<TO>(v[e]);
      }
    }
  }
}

template <typename TO, int BM, int BN>
__global__ void __launch_bounds__(256)
gemm_tile_kernel(const bf16_t* __restrict__ a, long lda, const bf16_t* __restrict__ w, const float* __restrict__ bias,
                 const float* residual, long ldr, TO* out, long ldo, int M, int N, int K, int act, int tiles_m, int tiles_n,
                 int vec_ok, int S, float* __restrict__ partial) {
  constexpr int WM = BM / 2, WN = BN / 2;    // the wave's tile
  constexpr int TI = WM / 32, TJ = WN / 32;  // in 32 x 32 MFMA tiles
  constexpr int CA = BM * (TK / 8) / 256;    // 16-byte chunks of the a tile per thread
  constexpr int CW = BN * (TK / 8) / 256;
  extern __shared__ __attribute__((aligned(16))) bf16_t smem[];
  bf16_t* As = smem;                               // [2][BM * LDS_STRIDE]
  bf16_t* Ws = smem + 2 * BM * LDS_STRIDE;         // [2][BN * LDS_STRIDE]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int n_tiles = tiles_m * tiles_n;
  int id = blockIdx.x;
  if (n_tiles % 8 == 0) id = (id % 8) * (n_tiles / 8) + id / 8;
  const int m0 = (id % tiles_m) * BM, n0 = (id / tiles_m) * BN;

  // Rows beyond the matrix read the last row instead: their products land in output rows / columns that are
  // never stored. Only the k range needs zeros, and the partial k-tile (K % 64 != 0) is taken FIRST, in the
  // prologue, so that the main loop needs no masks at all.
  uint32_t pa[CA], pw[CW];
  const int kc = (tid & 7) * 8;
#pragma unroll
  for (int i = 0; i < CA; ++i) pa[i] = (uint32_t)((size_t)min(m0 + ((tid + 256 * i) >> 3), M - 1) * lda);
#pragma unroll
  for (int i = 0; i < CW; ++i) pw[i] = (uint32_t)((size_t)min(n0 + ((tid + 256 * i) >> 3), N - 1) * K);
  // The k-tiles in the order they are taken: tile 0 is the partial one (K % 64 != 0) or the first, tile t >= 1 starts at
  // (t - kshift) * 64. With S > 1 (few output tiles: the K range is split over blockIdx.y) this workgroup takes
  // tiles t0 .. t1 - 1 and leaves its sums, without epilogue, in partial[blockIdx.y].
  const int ktail = K % TK, nk_all = (K + TK - 1) / TK;
  const int per = (nk_all + S - 1) / S;
  const int t0 = blockIdx.y * per, t1 = min(nk_all, t0 + per);
  const int nk = t1 - t0;
  const int kshift = ktail ? 1 : 0;
  auto kpos = [&](int t) {  // for t >= 1 (tiles past this range repeat its last one; they are loaded but never used)
    return max(min(t, t1 - 1) - kshift, 0) * TK;
  };
  u32x4 ra[2][CA], rw[2][CW];
  auto gload_one = [&](int set, uint32_t koff, int i) {
    if (i < CA) ra[set][i] = load16(a + pa[i] + koff);
    else rw[set][i - CA] = load16(w + pw[i - CA] + koff);
  };
  bf16_t* a_st = As + (tid >> 3) * LDS_STRIDE + kc;
  bf16_t* w_st = Ws + (tid >> 3) * LDS_STRIDE + kc;
  auto lstore_one = [&](int set, int buf, int i) {
    if (i < CA) *reinterpret_cast<u32x4*>(a_st + buf * BM * LDS_STRIDE + i * 32 * LDS_STRIDE) = ra[set][i];
    else *reinterpret_cast<u32x4*>(w_st + buf * BN * LDS_STRIDE + (i - CA) * 32 * LDS_STRIDE) = rw[set][i - CA];
  };

  f32x16 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  {  // prologue: this range's first tile (masked in k if it is the partial one) to LDS buffer 0, the next into register set 1
    const int k0 = t0 == 0 ? (ktail ? K - ktail : 0) : kpos(t0);
    const bool ok = k0 + kc < K;
    const uint32_t koff = (uint32_t)min(k0 + kc, K - 8);
#pragma unroll
    for (int i = 0; i < CA + CW; ++i) gload_one(0, koff, i);
#pragma unroll
    for (int i = 0; i < CA; ++i) if (!ok) ra[0][i] = u32x4{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < CW; ++i) if (!ok) rw[0][i] = u32x4{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < CA + CW; ++i) lstore_one(0, 0, i);
    const uint32_t koff1 = (uint32_t)min(kpos(t0 + 1) + kc, K - 8);
#pragma unroll
    for (int i = 0; i < CA + CW; ++i) gload_one(1, koff1, i);
  }
  lds_barrier();
  const int fr = lane & 31, fk = (lane >> 5) * 8;
  constexpr int KS = TK / 16;
  constexpr int NM = TI * TJ, NR = TI + TJ;
  constexpr int PW = (CA + CW + KS - 2) / (KS - 1);  // LDS writes / global loads per k-step, in the first KS - 1 k-steps
  const bf16_t* a_rd = As + (wm * WM + fr) * LDS_STRIDE + fk;
  const bf16_t* w_rd = Ws + (wn * WN + fr) * LDS_STRIDE + fk;
  u32x4 af[2][TI], wf[2][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i) af[0][i] = *reinterpret_cast<const u32x4*>(a_rd + i * 32 * LDS_STRIDE);
#pragma unroll
  for (int j = 0; j < TJ; ++j) wf[0][j] = *reinterpret_cast<const u32x4*>(w_rd + j * 32 * LDS_STRIDE);

  // One k-tile. `cur` is the register set that holds tile kt + 1 (it goes to the other LDS buffer during the
  // first KS - 1 k-steps); the other set receives the loads of tile kt + 2. Then one barrier, and the last
  // k-step's products cover the LDS reads of tile kt + 1's first fragments. Every product is followed by at
  // most two other instructions so that the matrix pipe never waits for the wave to issue them in a block.
  auto ktile = [&](int kt, int cur) {
    const int buf = kt & 1;
    const uint32_t koff = (uint32_t)min(kpos(t0 + kt + 2) + kc, K - 8);
    const bf16_t* Ab = a_rd + buf * BM * LDS_STRIDE;
    const bf16_t* Wb = w_rd + buf * BN * LDS_STRIDE;
    const bf16_t* Abn = a_rd + (buf ^ 1) * BM * LDS_STRIDE;
    const bf16_t* Wbn = w_rd + (buf ^ 1) * BN * LDS_STRIDE;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c = ks & 1, nx = c ^ 1;
      if (ks + 1 < KS) {
#pragma unroll
        for (int i = 0; i < TI; ++i) af[nx][i] = *reinterpret_cast<const u32x4*>(Ab + i * 32 * LDS_STRIDE + (ks + 1) * 16);
#pragma unroll
        for (int j = 0; j < TJ; ++j) wf[nx][j] = *reinterpret_cast<const u32x4*>(Wb + j * 32 * LDS_STRIDE + (ks + 1) * 16);
      } else {
        lds_barrier();
#pragma unroll
        for (int i = 0; i < TI; ++i) af[nx][i] = *reinterpret_cast<const u32x4*>(Abn + i * 32 * LDS_STRIDE);
#pragma unroll
        for (int j = 0; j < TJ; ++j) wf[nx][j] = *reinterpret_cast<const u32x4*>(Wbn + j * 32 * LDS_STRIDE);
      }
#pragma unroll
      for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(af[c][i]), as_bf16x8(wf[c][j]), acc[i][j], 0, 0, 0);
      if (ks + 1 < KS) {
#pragma unroll
        for (int q = 0; q < PW; ++q)
          if (ks * PW + q < CA + CW) lstore_one(cur, buf ^ 1, ks * PW + q);
#pragma unroll
        for (int q = 0; q < PW; ++q)
          if (ks * PW + q < CA + CW) gload_one(cur ^ 1, koff, ks * PW + q);
      }
      constexpr int others = NR + 2 * PW;
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (ks + 1 < KS) {
          const int lo = m * others / NM, hi = (m + 1) * others / NM;
#pragma unroll
          for (int o = lo; o < hi; ++o) {
            if (o < NR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            else if (o < NR + PW) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            else __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
          }
        } else {
          const int lo = m * NR / NM, hi = (m + 1) * NR / NM;
#pragma unroll
          for (int o = lo; o < hi; ++o) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
      }
    }
  };
  int kt = 0;
  for (; kt + 1 < nk; kt += 2) {
    ktile(kt, 1);
    ktile(kt + 1, 0);
  }
  if (kt < nk) ktile(kt, 1);

  // Epilogue (the operand buffers are free now), specialised for no activation and the two GELUs so that the
  // loop over the outputs has no switch inside
  lds_barrier();
  float* Cs = reinterpret_cast<float*>(smem) + wave * 32 * (BN / 2 + 4);
  const int mw = m0 + wm * WM, nw = n0 + wn * WN;
  if (S > 1)  // vec_ok: bit 1 says whether the partial sums can be stored as vectors
    tile_epilogue<float, LEV_ACT_NONE, TI, TJ>(acc, Cs, lane, mw, nw, nullptr, nullptr, 0, partial + (size_t)blockIdx.y * M * N, N, M, N,
                                               LEV_ACT_NONE, (vec_ok >> 1) & 1);
  else if (act == LEV_ACT_NONE)
    tile_epilogue<TO, LEV_ACT_NONE, TI, TJ>(acc, Cs, lane, mw, nw, bias, residual, ldr, out, ldo, M, N, act, vec_ok & 1);
  else if (act == LEV_ACT_GELU_TANH)
    tile_epilogue<TO, LEV_ACT_GELU_TANH, TI, TJ>(acc, Cs, lane, mw, nw, bias, residual, ldr, out, ldo, M, N, act, vec_ok & 1);
  else if (act == LEV_ACT_GELU_ERF)
    tile_epilogue<TO, LEV_ACT_GELU_ERF, TI, TJ>(acc, Cs, lane, mw, nw, bias, residual, ldr, out, ldo, M, N, act, vec_ok & 1);
  else
    tile_epilogue<TO, -1, TI, TJ>(acc, Cs, lane, mw, nw, bias, residual, ldr, out, ldo, M, N, act, vec_ok & 1);
}

// out = act(sum_s partial[s] + bias) + residual (defined with the stream kernel below)
template <typename TO>
static int launch_splitk_reduce(const float* workspace, const float* bias, const float* residual, long ldr, TO* out, long ldo, int M,
                                int N, int S, int act, hipStream_t stream);

template <typename TO, int BM, int BN>
static int launch_tile(const bf16_t* a, long lda, const bf16_t* w, const float* bias, const float* residual, long ldr, TO* out,
                       long ldo, float* workspace, int M, int N, int K, int act, int S, int defer, hipStream_t stream) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const size_t lds_ops = (size_t)2 * (BM + BN) * LDS_STRIDE * sizeof(bf16_t);
  const size_t lds_out = (size_t)4 * 32 * (BN / 2 + 4) * sizeof(float);
  const size_t lds = lds_ops > lds_out ? lds_ops : lds_out;
  static bool configured = false;  // per instantiation
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_tile_kernel<TO, BM, BN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return lev_fail("linear: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    configured = true;
  }
  if (S > 1 && !workspace) return lev_fail("linear: M=%d N=%d K=%d needs a workspace of lev_linear_mfma_workspace bytes", M, N, K);
  // rows of 4 outputs are stored (and bias / residual read) as vectors when everything is aligned for it
  const int vec_out = (ldo % 4 == 0) && (((uintptr_t)out & 15) == 0) && (!residual || (ldr % 4 == 0 && ((uintptr_t)residual & 15) == 0)) &&
                      (!bias || ((uintptr_t)bias & 15) == 0);
  const int vec_partial = (N % 4 == 0) && (((uintptr_t)workspace & 15) == 0);
  gemm_tile_kernel<TO, BM, BN><<<dim3(tiles_m * tiles_n, S), 256, lds, stream>>>(a, lda, w, bias, residual, ldr, out, ldo, M, N, K, act,
                                                                                   tiles_m, tiles_n, vec_out | (vec_partial << 1), S,
                                                                                   workspace);
  if (S > 1) {
    if (int rc = lev_check_launch("linear_tile")) return rc;
    if (defer) return 0;  // the caller folds the sum of the ranges into its next kernel
    return launch_splitk_reduce<TO>(workspace, bias, residual, ldr, out, ldo, M, N, S, act, stream);
  }
  return 0;
}

// ------------------------------------------------------------------------------------------------
// Skinny kernel (M <= SKINNY_MAX_M: MT = 1, 2 or 4 tiles of 16 rows). A workgroup owns NT = 1 to 3 units of 16 output columns; its WAVES
// waves split K. A wave takes pairs of adjacent 32-wide k-steps (64 k = 128 bytes of a row), U pairs in flight:
//   weights: lane (row l%16, k-group l/16) loads 16 bytes straight into the MFMA operand, two loads per pair;
//   `a`:     read as WHOLE 128-byte lines - lane (row l/8, 16-byte chunk l%8), one instruction for rows 0..7 and one
//            for rows 8..15 of a pair - and turned into the operand layout (row l%16, k-group l/16) through a
//            small LDS area of the wave's own. Reading `a` in operand layout (64 bytes of each of 16 rows per
//            instruction) costs as much time in the memory pipeline as the weights themselves: every workgroup
//            reads all of `a`, and half lines are fetched at half the rate.
// The partial sums of the waves are added through LDS in wave order. ROT: every workgroup starts at another
// place of the k range, so that they do not all read the same part of `a` and the same residue of the weight
// rows at the same time; the order of the sum depends on the column tile only, never on M or the batch.
#define SKINNY_SLOTS 72  // 16-byte slots of one staged instruction: 8 rows x (8 chunks + 1 of padding)
#define SKINNY_MAX_M 64  // with four row tiles; which of these row counts it takes: use_skinny()

template <typename TO, int WAVES, int U, int ROT, int MT, int NT>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ a, long lda, const bf16_t* __restrict__ w, const float* __restrict__ bias,
                   const float* residual, long ldr, TO* out, long ldo, int M, int N, int K, int act) {
  static_assert(NT >= 1 && NT <= WAVES, "wave j finishes column unit j");
  constexpr int AI = 2 * MT;  // `a` instructions per pair of k-steps: 8 rows each
  // With more than two row tiles the staging area holds one tile at a time (the LDS executes a wave's instructions in
  // order, so the next tile's writes cannot overtake this one's reads): 16 waves x 8 instructions would not fit the LDS.
  constexpr bool ONE_TILE = MT > 2;
  constexpr int SI = ONE_TILE ? 2 : AI;
  __shared__ f32x4 red[WAVES][NT][MT][64];
  __shared__ u32x4 stage[WAVES][SI][SKINNY_SLOTS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * 16 * NT;
  const int fr = lane & 15, kg = lane >> 4;
  bool n_ok[NT];
  const bf16_t* wrow[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    n_ok[j] = n0 + 16 * j + fr < N;
    wrow[j] = w + (size_t)(n_ok[j] ? n0 + 16 * j + fr : 0) * K + kg * 8;
  }
  const int ar = lane >> 3, ac = lane & 7;  // `a` loads: row (0..7, instruction i adds 8 i) and chunk of the line
  bool a_ok[AI];
  const bf16_t* arow[AI];
#pragma unroll
  for (int i = 0; i < AI; ++i) {
    a_ok[i] = ar + 8 * i < M;
    arow[i] = a + (size_t)(a_ok[i] ? ar + 8 * i : 0) * lda + ac * 8;
  }
  u32x4* my_stage = &stage[wave][0][0];
  const int st_slot = ar * 9 + ac;                       // where this lane's chunk is staged
  const int ld_slot = (fr >> 3) * SKINNY_SLOTS + (fr & 7) * 9 + kg;  // operand (row fr, k-group kg) of the pair's first step

  // The lanes that will finish the sum fetch their bias and residual values now, so that the end of the kernel
  // (which no other workgroup's streaming overlaps: all of them finish together) has no dependent loads left.
  // Unconditional loads from addresses that are always valid (clamped; `w` stands in for a missing operand):
  // a load under a condition would make the compiler wait for it at the join, ahead of the whole k loop.
  float pre_bias[NT];
  f32x4 pre_res[NT][MT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int nn = min(n0 + 16 * j + fr, N - 1);
    const float* bp = bias ? bias + nn : reinterpret_cast<const float*>(w);
    pre_bias[j] = *bp;
    if (!bias) pre_bias[j] = 0.f;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = min(t * 16 + kg * 4 + r, M - 1);
        const float* rp = residual ? residual + (size_t)m * ldr + nn : reinterpret_cast<const float*>(w);
        pre_res[j][t][r] = *rp;
      }
  }

  f32x4 acc[NT][MT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[j][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int npairs = (K + 63) / 64;
  const int rot = ROT ? (int)((blockIdx.x * 2654435761u) % (unsigned)npairs) : 0;
  for (int p0 = wave; p0 < npairs; p0 += WAVES * U) {
    u32x4 wv[U][NT][2], av[U][AI];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int pr = p0 + u * WAVES;
      const bool p_ok = pr < npairs;
      if (ROT) {
        pr += rot;
        pr = pr >= npairs ? pr - npairs : pr;
      }
      const int k = pr * 64;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const bool w_ok = p_ok && n_ok[j];
        wv[u][j][0] = (w_ok && k + kg * 8 < K) ? load16(wrow[j] + k) : u32x4{0, 0, 0, 0};
        wv[u][j][1] = (w_ok && k + 32 + kg * 8 < K) ? load16(wrow[j] + k + 32) : u32x4{0, 0, 0, 0};
      }
      const bool c_ok = p_ok && k + ac * 8 < K;
#pragma unroll
      for (int i = 0; i < AI; ++i) av[u][i] = (c_ok && a_ok[i]) ? load16(arow[i] + k) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // LDS executes a wave's instructions in order: the area is reused pair after pair without a barrier
      if (!ONE_TILE) {
#pragma unroll
        for (int i = 0; i < AI; ++i) my_stage[i * SKINNY_SLOTS + st_slot] = av[u][i];
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if (ONE_TILE) {
          my_stage[st_slot] = av[u][2 * t];
          my_stage[SKINNY_SLOTS + st_slot] = av[u][2 * t + 1];
        }
        const int base = ONE_TILE ? 0 : 2 * t * SKINNY_SLOTS;
        const u32x4 a_lo = my_stage[base + ld_slot], a_hi = my_stage[base + ld_slot + 4];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a_lo), as_bf16x8(wv[u][j][0]), acc[j][t], 0, 0, 0);
          acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a_hi), as_bf16x8(wv[u][j][1]), acc[j][t], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int t = 0; t < MT; ++t) red[wave][j][t][lane] = acc[j][t];
  __syncthreads();
  // 16x16 accumulator: register r of lane l is row 4*(l/16) + r, column l%16. Partial sums are added in wave order.
  if (wave < NT) {  // wave j finishes column unit j
    const int j = wave;
    const int nn = n0 + 16 * j + fr;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      f32x4 s = red[0][j][t][lane];
#pragma unroll
      for (int v = 1; v < WAVES; ++v) {
        const f32x4 o = red[v][j][t][lane];
        s[0] += o[0]; s[1] += o[1]; s[2] += o[2]; s[3] += o[3];
      }
      if (nn < N) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = t * 16 + kg * 4 + r;
          if (m >= M) continue;
          float pb = pre_bias[0], pr = pre_res[0][t][r];
#pragma unroll
          for (int j2 = 1; j2 < NT; ++j2)
            if (j == j2) {
              pb = pre_bias[j2];
              pr = pre_res[j2][t][r];
            }
          float v = lev_activate(s[r] + pb, act);
          if (residual) v += pr;
          out[(size_t)m * ldo + nn] = from_float<TO>(v);
        }
      }
    }
  }
}

// Choices measured on MI355X at K = 4096 .. 16384 and M = 1 .. 16 (graph replays over distinct weights): with many
// column tiles 4 waves with 4 or 2 pairs in flight; with fewer than 512 the chip is only filled by 16 waves per
// workgroup. The rotated start never costs and takes a third off the time where rows are long (K = 16384).
// Two column units per workgroup (32 columns: every `a` fragment feeds two weight fragments, half the activation
// traffic) pay where the halved number of workgroups still fills the chip evenly or the rows are many: 16384
// columns x 4096 at 8 rows 28.1 -> 26.2 us, at 16 rows 33.4 -> 27.8 us; 24576 x 6144 at 16 rows 76 -> 64 us; at one
// row and with workgroup counts that are no multiple of the CUs (18432 or 50257 columns) they lose up to 15 %.
// Three units and 16 waves for 12288 columns x 4096: 25.1 -> 21.8 us at 16 rows, the same at 8 rows, 10 % slower at one.
struct SkinnyShape {
  int waves, in_flight, row_tiles, units;  // the kernel's WAVES, U, MT, NT
};
static SkinnyShape skinny_shape(int M, int N) {
  const int tiles = (N + 15) / 16;
  if (M <= 16) {
    const bool two_units = tiles >= 1024 && (M >= 12 || (tiles / 2) % 256 == 0);
    if (two_units) return {4, 2, 1, 2};
    if (M >= 12 && tiles >= 720 && tiles < 1024) return {16, 1, 1, 3};  // about 256 workgroups of 48 columns
    if (tiles >= 1024) return {4, 4, 1, 1};
    if (tiles >= 512) return {4, 2, 1, 1};
    return {16, 1, 1, 1};
  }
  // 17 .. 32 rows: two row tiles share every weight load; up to SKINNY_MAX_M: four
  if (M <= 32) return tiles >= 512 ? SkinnyShape{4, 2, 2, 1} : SkinnyShape{16, 1, 2, 1};
  return tiles >= 512 ? SkinnyShape{4, 2, 4, 1} : SkinnyShape{16, 1, 4, 1};
}

template <typename TO>
static void launch_skinny(const bf16_t* a, long lda, const bf16_t* w, const float* bias, const float* residual, long ldr,
                          TO* out, long ldo, int M, int N, int K, int act, hipStream_t stream) {
  const int tiles = (N + 15) / 16;
  const SkinnyShape sh = skinny_shape(M, N);
#define LEV_SKINNY(W_, U_, MT_, NT_)                                                                                          \
  if (sh.waves == W_ && sh.in_flight == U_ && sh.row_tiles == MT_ && sh.units == NT_)                                          \
    gemm_skinny_kernel<TO, W_, U_, 1, MT_, NT_><<<(tiles + NT_ - 1) / NT_, W_ * 64, 0, stream>>>(a, lda, w, bias, residual, ldr, out, \
                                                                                                 ldo, M, N, K, act)
  LEV_SKINNY(4, 2, 1, 2);
  LEV_SKINNY(16, 1, 1, 3);
  LEV_SKINNY(4, 4, 1, 1);
  LEV_SKINNY(4, 2, 1, 1);
  LEV_SKINNY(16, 1, 1, 1);
  LEV_SKINNY(4, 2, 2, 1);
  LEV_SKINNY(16, 1, 2, 1);
  LEV_SKINNY(4, 2, 4, 1);
  LEV_SKINNY(16, 1, 4, 1);
#undef LEV_SKINNY
}

// ------------------------------------------------------------------------------------------------
// Stream kernel, for 24 < M <= 128: the weights are still the traffic that matters, but fetching the `a`
// fragments from L2 once per wave (as the skinny kernel does) would cost more than the weights. Here a
// workgroup of NW waves (4, 8, 12 or 16) owns NW x 16 output columns and all M rows; `a` goes through LDS in chunks
// of 64 k and is shared by the waves, each wave loads its own 16 weight rows straight into MFMA operand
// registers. To fill the chip the K range is split over `S` workgroups (blockIdx.y); with S > 1 the partial
// sums go to a float32 workspace [S][M][N] and a second kernel adds them in order and applies the epilogue.
#define SK_CHUNK 64
#define SK_LDS_STRIDE (SK_CHUNK + 8)

template <typename TO, int MT, int NW>
__global__ void __launch_bounds__(NW * 64)
gemm_stream_kernel(const bf16_t* __restrict__ a, long lda, const bf16_t* __restrict__ w, const float* __restrict__ bias,
                   const float* residual, long ldr, TO* out, long ldo, float* __restrict__ partial, int M, int N, int K, int act,
                   int S) {
  constexpr int BM = MT * 16;
  constexpr int NT = NW * 64;
  constexpr int A_CHUNKS = BM * (SK_CHUNK / 8);       // 16-byte chunks of the a tile
  constexpr int XCH = (A_CHUNKS + NT - 1) / NT;       // per thread (threads beyond the tile repeat its last chunk)
  __shared__ __attribute__((aligned(16))) bf16_t Xs[2][BM * SK_LDS_STRIDE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int fr = lane & 15, fk = (lane >> 4) * 8;
  const int n0 = blockIdx.x * (NW * 16) + wave * 16;
  const int split = blockIdx.y;
  const int n_chunks = (K + SK_CHUNK - 1) / SK_CHUNK;
  const int per = (n_chunks + S - 1) / S;
  const int c_begin = split * per, c_end = min(n_chunks, c_begin + per);
  const int n = n0 + fr;
  const bf16_t* wrow = w + (size_t)min(n, N - 1) * K;  // a row beyond N reads the last one; its column is never stored
  // this thread's chunks of the a tile
  uint32_t xoff[XCH];
  int xk[XCH], xlds[XCH];
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int c = min(tid + NT * i, A_CHUNKS - 1);
    const int row = c / (SK_CHUNK / 8);
    xk[i] = (c % (SK_CHUNK / 8)) * 8;
    xoff[i] = (uint32_t)((size_t)min(row, M - 1) * lda);
    xlds[i] = row * SK_LDS_STRIDE + xk[i];
  }
  // two register sets for the a tile as for the weights: a chunk's loads are issued two iterations before it is
  // stored to LDS. With one set an iteration could not be shorter than the L2 latency of the a loads of the
  // iteration before (about a microsecond, where its own work is a few hundred cycles).
  u32x4 xr[2][XCH];
  constexpr int KS = SK_CHUNK / 32;  // k-steps per chunk
  u32x4 wr[2][KS];
  auto load_x = [&](int set, int c) {
    const int k0 = min(c, n_chunks - 1) * SK_CHUNK;
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int k = k0 + xk[i];
      xr[set][i] = load16(a + xoff[i] + (k < K ? k : K - 8));
    }
  };
  auto store_x = [&](int buf, int set, int c) {
    const int k0 = c * SK_CHUNK;
#pragma unroll
    for (int i = 0; i < XCH; ++i)
      *reinterpret_cast<u32x4*>(&Xs[buf][xlds[i]]) = (k0 + xk[i] < K) ? xr[set][i] : u32x4{0, 0, 0, 0};
  };
  auto load_w = [&](int set, int c) {
    const int k0 = min(c, n_chunks - 1) * SK_CHUNK;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int k = k0 + s * 32 + fk;
      wr[set][s] = load16(wrow + (k < K ? k : K - 8));  // beyond K the a fragment is zero, whatever this holds
    }
  };
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (c_begin < c_end) {
    load_x(0, c_begin);
    load_w(0, c_begin);
    load_x(1, c_begin + 1);
    load_w(1, c_begin + 1);
    store_x(0, 0, c_begin);
    load_x(0, c_begin + 2);
    lds_barrier();
    // chunk c (weights in set `set`, a tile in LDS buffer `set`): the a tile of chunk c + 1, in registers since the
    // iteration before last, goes to the other buffer; its registers are refilled three chunks ahead, this chunk's
    // weight registers two chunks ahead
    auto chunk = [&](int c, int set) {
      store_x(set ^ 1, set ^ 1, c + 1);  // past this split's last chunk it fills the buffer nobody reads
      load_x(set ^ 1, c + 3);
      const bf16_t* xb = &Xs[set][fr * SK_LDS_STRIDE + fk];
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const u32x4 af = *reinterpret_cast<const u32x4*>(xb + t * 16 * SK_LDS_STRIDE + s * 32);
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(af), as_bf16x8(wr[set][s]), acc[t], 0, 0, 0);
        }
      // the weight registers are refilled behind the products that read them: refilled ahead of them (from a copy),
      // the new values landed in other registers and were moved into place at the end of the loop, which waits for
      // loads issued a moment before
      load_w(set, c + 2);
      lds_barrier();
      // Nothing moves across the end of a chunk: the compiler had lifted the next chunk's masking of its a registers
      // (a select per register) to the top of the loop, where it waited for every load in flight, the weights
      // requested a moment before among them, and each pair of chunks cost a whole memory latency.
      __builtin_amdgcn_sched_barrier(0);
    };
    int c = c_begin;
    for (; c + 1 < c_end; c += 2) {
      chunk(c, 0);
      chunk(c + 1, 1);
    }
    if (c < c_end) chunk(c, 0);
  }
  // 16x16 accumulator: register r of lane l is row 4*(l/16) + r, column l%16
  if (n < N) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = t * 16 + (lane >> 4) * 4 + r;
        if (m < M) {
          if (S == 1)
            epilogue_store<TO>(acc[t][r], m, n, bias, residual, ldr, out, ldo, act);
          else
            partial[((size_t)split * M + m) * N + n] = acc[t][r];
        }
      }
  }
}

// out = act(sum_s partial[s] + bias) + residual, the partial sums added in the order of s.
// VEC: four consecutive columns per thread (N a multiple of 4 and every pointer and row stride aligned for it).
template <typename TO, int VEC>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float* __restrict__ partial, const float* __restrict__ bias, const float* residual, long ldr, TO* out,
                     long ldo, int M, int N, int S, int act) {
  const size_t total = (size_t)M * N;
  const size_t idx = ((size_t)blockIdx.x * 256 + threadIdx.x) * (VEC ? 4 : 1);
  if (idx >= total) return;
  const int m = (int)(idx / N), n = (int)(idx % N);
  if (VEC) {
    // four ranges are requested at once and added in their order: a loop of load - add - load paid the latency of
    // every range in turn (the partial sums come from other CUs, out of L2 at best)
    f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
    const float* src = partial + idx;
    int s = 0;
    for (; s + 4 <= S; s += 4) {
      f32x4 p[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) p[j] = *reinterpret_cast<const f32x4*>(src + (size_t)(s + j) * total);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[0] += p[j][0]; v[1] += p[j][1]; v[2] += p[j][2]; v[3] += p[j][3];
      }
    }
    {
      f32x4 p[3];
#pragma unroll
      for (int j = 0; j < 3; ++j)  // the last ranges, unconditionally from a valid place
        p[j] = *reinterpret_cast<const f32x4*>(src + (size_t)min(s + j, S - 1) * total);
#pragma unroll
      for (int j = 0; j < 3; ++j)
        if (s + j < S) {
          v[0] += p[j][0]; v[1] += p[j][1]; v[2] += p[j][2]; v[3] += p[j][3];
        }
    }
    float o[4] = {v[0], v[1], v[2], v[3]};
    if (bias) {
      const f32x4 b = *reinterpret_cast<const f32x4*>(bias + n);
      o[0] += b[0]; o[1] += b[1]; o[2] += b[2]; o[3] += b[3];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = lev_activate(o[e], act);
    if (residual) {
      const f32x4 r = *reinterpret_cast<const f32x4*>(residual + (size_t)m * ldr + n);
      o[0] += r[0]; o[1] += r[1]; o[2] += r[2]; o[3] += r[3];
    }
    store_vec4<TO>(out + (size_t)m * ldo + n, o);
  } else {
    float v = 0.f;
    for (int s = 0; s < S; ++s) v += partial[(size_t)s * total + idx];
    epilogue_store<TO>(v, m, n, bias, residual, ldr, out, ldo, act);
  }
}

template <typename TO>
static int launch_splitk_reduce(const float* workspace, const float* bias, const float* residual, long ldr, TO* out, long ldo, int M,
                                int N, int S, int act, hipStream_t stream) {
  const size_t total = (size_t)M * N;
  const bool vec = (N % 4 == 0) && (ldo % 4 == 0) && (((uintptr_t)out & 15) == 0) && (((uintptr_t)workspace & 15) == 0) &&
                   (!residual || (ldr % 4 == 0 && ((uintptr_t)residual & 15) == 0)) && (!bias || ((uintptr_t)bias & 15) == 0);
  if (vec)
    splitk_reduce_kernel<TO, 1><<<(unsigned)((total / 4 + 255) / 256), 256, 0, stream>>>(workspace, bias, residual, ldr, out, ldo, M, N, S,
                                                                                          act);
  else
    splitk_reduce_kernel<TO, 0><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(workspace, bias, residual, ldr, out, ldo, M, N, S, act);
  return lev_check_launch("linear_reduce");
}

// The shape of the stream kernel's launch: how many waves a workgroup has (16 columns each) and into how many k ranges
// K is split. An estimate in microseconds of every combination, fitted to measurements on MI355X of weights from
// 5 MB to 400 MB at 32 to 128 rows.
//   What the CUs fetch is the weights once and the activations once per column tile: a wider workgroup shares its a
//     tile among more columns (at 64 rows and 64 columns the a tiles are as many bytes as the weights). Together
//     the CUs get about 7.5 TB/s out of L2.
//   A CU holds 16 waves of this kernel. The slowest CU has r = ceil(workgroups / 256) workgroups and takes r times a
//     workgroup's share of that time, plus about a microsecond each. With 4 or 8 waves on a CU the loads in flight do
//     not cover the memory latency (x 1.45, x 1.12); 12 or 16 do.
//   More than one range: the second kernel's launch (3 us) and the partial sums, M x N floats per range that are
//     written and read again (4 S M / K of the weights' bytes, mostly out of the caches: weighted half).
//   Measured at the 7B sizes, 64 rows (qkv / proj / fc / mproj, second kernel included): 4 waves 33 / 18 / 42 / 43 us,
//     the shapes chosen here (12 x 4 ranges, 12 x 11, 16 x 4, 16 x 16) 29 / 17 / 40 / 38 us; at 128 rows 47 / 20 / 58 / 55
//     against 37 / 22 / 46 / 45 us.
struct StreamPlan {
  int waves;   // waves of a workgroup (16 columns each): 4, 8, 12 or 16
  int splits;  // k ranges
  double cost; // the estimate, in the model's microseconds
};
static StreamPlan plan_stream(int M, int N, int K) {
  static const int nw[4] = {4, 8, 12, 16};
  const int chunks = (K + SK_CHUNK - 1) / SK_CHUNK;
  const int s_max = chunks / 2 < 16 ? (chunks / 2 < 1 ? 1 : chunks / 2) : 16;  // at least two chunks each
  const double w_bytes = (double)N * K * 2.0;
  StreamPlan best = {4, 1, 1e30};
  double best_cost = 1e30;
  const int n_widths = w_bytes < 24e6 ? 1 : 4;  // weights of a few MB: the narrow workgroup measured best throughout
  for (int i = 0; i < n_widths; ++i) {
    const int tiles = (N + nw[i] * 16 - 1) / (nw[i] * 16);
    const int per_cu = 16 / nw[i];  // workgroups that stay on a CU at once
    const double a_bytes = (double)tiles * M * K * 2.0;  // every column tile reads all of a, once over its ranges
    for (int s = 1; s <= s_max; ++s) {
      const long wgs = (long)tiles * s;
      const long r = (wgs + 255) / 256;  // workgroups of the slowest CU
      if (r > per_cu && wgs > 256L * per_cu) continue;
      const int waves_cu = (int)r * nw[i];
      const double latency = waves_cu <= 4 ? 1.45 : (waves_cu <= 8 ? 1.12 : 1.0);
      const double t = (w_bytes + a_bytes) / 7.5e6;  // microseconds at what the CUs get out of L2 together
      double cost = (double)r * (1.0 + t * 256.0 / wgs * latency);
      if (s > 1) cost += 3.0 + 2.0 * s * M / K * (w_bytes / 4.5e6);
      if (cost < best_cost - 1e-9) {
        best_cost = cost;
        best = {nw[i], s, cost};
      }
    }
  }
  return best;
}

// Tile shape and number of k ranges for M > 128. Estimated time of each tile shape: rounds of workgroups over the 256
// CUs times (k-tiles x the shape's time per k-tile + a fixed cost for a tile's first loads and its epilogue). Two
// 128 x 128 workgroups fit a CU and then share it; up to 256 of them have a CU each. Where the output has so few
// tiles that most CUs would idle (a few hundred rows times a narrow weight), K is split into ranges, as in the
// stream kernel: the second kernel then costs its launch and the traffic of the partial sums. The constants are
// microseconds measured on MI355X.
struct TilePlan {
  int shape;   // 0: 256 x 256, 1: 256 x 192, 2: 256 x 128, 3: 128 x 128, 4: 128 x 64
  int splits;  // k ranges (1: none)
};
static TilePlan plan_tiles(int M, int N, int K) {
  static const int bm[5] = {256, 256, 256, 128, 128}, bn[5] = {256, 192, 128, 128, 64};
  static const double us_per_ktile[5] = {1.72, 1.36, 0.97, 0.6, 0.4}, fixed[5] = {13.0, 11.0, 9.0, 7.0, 6.0};
  const long nk = (K + TK - 1) / TK;
  TilePlan best = {0, 1};
  double best_cost = 1e30;
  for (int i = 0; i < 5; ++i) {
    const long tiles = (long)((M + bm[i] - 1) / bm[i]) * ((N + bn[i] - 1) / bn[i]);
    double cost;
    if (i == 4 && tiles > 256)
      continue;  // the small tile is for outputs that would leave CUs idle otherwise
    else if (i == 3 && tiles > 256)
      cost = (double)((tiles + 511) / 512) * (nk * 1.05 + 9.0);
    else
      cost = (double)((tiles + 255) / 256) * (nk * us_per_ktile[i] + fixed[i]);
    if (cost < best_cost) {
      best_cost = cost;
      best = {i, 1};
    }
    for (int s = 2; s <= 16 && tiles * s <= 256 && nk / s >= 4; ++s) {
      const long per = (nk + s - 1) / s;
      if (per * (s - 1) >= nk) continue;  // a range would be empty
      const double reduce = 4.0 + (double)(s + 1) * M * N * 4.0 / 3.0e6;
      const double c = per * us_per_ktile[i] + fixed[i] + reduce;
      if (c < best_cost) {
        best_cost = c;
        best = {i, s};
      }
    }
  }
  return best;
}

// Which kernel takes M <= SKINNY_MAX_M rows. The skinny kernel's time grows with the rows, because every workgroup reads all
// of `a` (out of L2, at about 20 TB/s for all CUs together), and with workgroup counts that are no multiple of the CUs; the
// stream kernel's hardly does, but it pays for its K ranges. An estimate of the skinny kernel in the manner of
// plan_stream's, and a factor between the two fitted to measurements at three model sizes (microseconds, skinny / stream):
//   4096-wide layer:  8 rows 19.5 / 24.1, 8.6 / 14.7, 24.9 / 31.6, 23.9 / 32.9 (qkv, proj, fc, second MLP matrix);
//                     24 rows 27.8 / 25.2, 12.6 / 15.9, 35.8 / 33.2, 35.3 / 33.6
//   6144-wide layer:  8 rows 48.3 / 53.7, 20.6 / 21.4, 55.2 / 59.2, 67.0 / 60.3; 16 rows 55.3 / 54.5, 25.0 / 22.0, 60.3 / 60.3,
//                     86.1 / 60.6 (384 workgroups of the skinny kernel: one and a half rounds); 24 rows 66 / 55, 32 / 23, 80 / 62, 104 / 62
//   1600-wide layer:  8 rows 7.0 / 8.1, 4.7 / 7.1, 8.3 / 9.5, 10.8 / 10.8; 16 rows 7.3 / 8.2, 4.8 / 7.2, 9.0 / 10.0, 13.6 / 11.0
//   heads (50257 columns) of 4096 / 6144 / 1600 / 768: 8 rows 81 / 87, 125 / 152, 34.6 / 34.3, 17.0 / 20.6; 24 rows 108 / 91, 169 / 156,
//                     46.5 / 35.9, 24.3 / 22.2
// Over the 112 cases measured (1 to 24 rows) the choice made here is on average 1 % behind the better kernel; the rule before
// it (rows alone, with one exception for large weights) 4 %, and up to 70 % on the long sums of the 6144-wide layer.
static double skinny_estimate(int M, int N, int K) {
  const SkinnyShape sh = skinny_shape(M, N);
  const long wgs = ((N + 15) / 16 + sh.units - 1) / sh.units;
  const long r = (wgs + 255) / 256;  // workgroups of the slowest CU
  const double w_bytes = (double)N * K * 2.0, a_bytes = (double)wgs * M * K * 2.0;
  const double t = w_bytes / 7.5e6 + a_bytes / 20e6;
  double cost = 3.0 + t * (wgs >= 256 ? (double)r * 256.0 / wgs : 256.0 / wgs);
  if (sh.row_tiles == 2) cost *= 1.2;
  return cost;
}
// 0: the estimate decides; 1 / 2: the skinny / the stream kernel wherever it takes the row count. For measurements of the
// choice itself (a test times both candidates at widths the estimates were not fitted to); not used by the engine.
static int g_force_kernel = 0;
extern "C" int lev_linear_mfma_force(int kind) {
  LEV_REQUIRE(kind >= 0 && kind <= 2, "linear: unknown kernel choice %d (0: by estimate, 1: skinny, 2: stream)", kind);
  g_force_kernel = kind;
  return 0;
}
static bool use_skinny(int M, int N, int K) {
  if (M > SKINNY_MAX_M) return false;
  if (g_force_kernel) return g_force_kernel == 1;
  if (M > 24) {
    // 25 to 64 rows (two or four row tiles), microseconds skinny / stream, second kernel included, at 32 and 64 rows: where
    // the skinny kernel's workgroups of 16 waves make one round of the CUs and the sum is no longer than the output is wide
    // it stays ahead (2304 x 768: 5.2 / 7.6, 7.6 / 9.4; 4096 x 1024: 6.1 / 8.6, 8.9 / 10.4; 1600 x 1600: 6.5 / 8.4, 9.5 / 10.2;
    // 4096 x 4096: 13.4 / 15.0 but 18.6 / 16.7), elsewhere not (4800 x 1600, 300 workgroups: 14.1 / 11.1, 20.4 / 13.4;
    // 1024 x 4096: 11.4 / 9.3, 16.2 / 11.0; 12288 x 4096: 32.1 / 26.4, 42.4 / 28.7).
    const int tiles = (N + 15) / 16;
    return tiles <= 256 && K <= N && (M <= 32 || (long)N * K <= (1L << 23));
  }
  return skinny_estimate(M, N, K) <= 1.3 * plan_stream(M, N, K).cost;
}

// Into how many ranges the sum over K is split (1: the kernel finishes its outputs itself).
extern "C" int lev_linear_mfma_ranges(int M, int N, int K) {
  if (use_skinny(M, N, K)) return 1;
  return M <= 128 ? plan_stream(M, N, K).splits : plan_tiles(M, N, K).splits;
}

extern "C" long lev_linear_mfma_workspace(int M, int N, int K) {
  const int S = lev_linear_mfma_ranges(M, N, K);
  return S > 1 ? (long)S * M * N * (long)sizeof(float) : 0;
}

// out = act(sum of the S ranges in workspace [S][M][N] + bias) + residual: what lev_linear_mfma runs itself unless it was
// asked to leave the ranges to the caller.
extern "C" int lev_linear_mfma_finish(const float* workspace, const float* bias, const float* residual, long ldr, void* out, long ldo,
                                      int M, int N, int S, int act, int out_dtype, hipStream_t stream) {
  LEV_REQUIRE(workspace && M > 0 && N > 0 && S > 1, "linear: nothing to finish (M=%d N=%d ranges=%d)", M, N, S);
  if (out_dtype == LEV_F32) return launch_splitk_reduce<float>(workspace, bias, residual, ldr, (float*)out, ldo, M, N, S, act, stream);
  if (out_dtype == LEV_BF16) return launch_splitk_reduce<bf16_t>(workspace, bias, residual, ldr, (bf16_t*)out, ldo, M, N, S, act, stream);
  return lev_fail("linear: unknown output dtype %d", out_dtype);
}

template <typename TO>
static int launch_stream(const bf16_t* a, long lda, const bf16_t* w, const float* bias, const float* residual, long ldr, TO* out,
                         long ldo, float* workspace, int M, int N, int K, int act, int defer, hipStream_t stream) {
  if ((size_t)M * lda >= (1ull << 32)) return lev_fail("linear: the activation matrix is too large (M=%d lda=%ld)", M, lda);
  const StreamPlan plan = plan_stream(M, N, K);
  const int S = plan.splits;
  if (S > 1 && !workspace) return lev_fail("linear: M=%d N=%d K=%d needs a workspace of lev_linear_mfma_workspace bytes", M, N, K);
  dim3 grid((N + plan.waves * 16 - 1) / (plan.waves * 16), S);
#define LEV_STREAM(MT_, NW_) \
  gemm_stream_kernel<TO, MT_, NW_><<<grid, NW_ * 64, 0, stream>>>(a, lda, w, bias, residual, ldr, out, ldo, workspace, M, N, K, act, S)
#define LEV_STREAM_MT(MT_)                 \
  switch (plan.waves) {                    \
    case 4: LEV_STREAM(MT_, 4); break;     \
    case 8: LEV_STREAM(MT_, 8); break;     \
    case 12: LEV_STREAM(MT_, 12); break;   \
    default: LEV_STREAM(MT_, 16); break;   \
  }
  if (M <= 32) {
    LEV_STREAM_MT(2)
  } else if (M <= 64) {
    LEV_STREAM_MT(4)
  } else {
    LEV_STREAM_MT(8)
  }
#undef LEV_STREAM_MT
#undef LEV_STREAM
  if (int rc = lev_check_launch("linear_stream")) return rc;
  if (S > 1 && !defer) return launch_splitk_reduce<TO>(workspace, bias, residual, ldr, out, ldo, M, N, S, act, stream);
  return 0;
}

template <typename TO>
static int linear_mfma_typed(const bf16_t* a, long lda, const bf16_t* w, const float* bias, const float* residual, long ldr,
                             TO* out, long ldo, float* workspace, int M, int N, int K, int act, int defer, hipStream_t stream) {
  if (use_skinny(M, N, K)) {
    launch_skinny<TO>(a, lda, w, bias, residual, ldr, out, ldo, M, N, K, act, stream);
  } else if (M <= 128) {
    return launch_stream<TO>(a, lda, w, bias, residual, ldr, out, ldo, workspace, M, N, K, act, defer, stream);
  } else {
    if ((size_t)M * lda >= (1ull << 31) || (size_t)N * K >= (1ull << 31))
      return lev_fail("linear: operands of more than 2^31 elements are not supported (M=%d lda=%ld N=%d K=%d)", M, lda, N, K);
    const TilePlan plan = plan_tiles(M, N, K);
    int rc;
    if (plan.shape == 0)
      rc = launch_tile<TO, 256, 256>(a, lda, w, bias, residual, ldr, out, ldo, workspace, M, N, K, act, plan.splits, defer, stream);
    else if (plan.shape == 1)
      rc = launch_tile<TO, 256, 192>(a, lda, w, bias, residual, ldr, out, ldo, workspace, M, N, K, act, plan.splits, defer, stream);
    else if (plan.shape == 2)
      rc = launch_tile<TO, 256, 128>(a, lda, w, bias, residual, ldr, out, ldo, workspace, M, N, K, act, plan.splits, defer, stream);
    else if (plan.shape == 3)
      rc = launch_tile<TO, 128, 128>(a, lda, w, bias, residual, ldr, out, ldo, workspace, M, N, K, act, plan.splits, defer, stream);
    else
      rc = launch_tile<TO, 128, 64>(a, lda, w, bias, residual, ldr, out, ldo, workspace, M, N, K, act, plan.splits, defer, stream);
    if (rc) return rc;
  }
  return lev_check_launch("linear_mfma");
}

// leave_ranges: where the sum over K is split into ranges (lev_linear_mfma_ranges > 1) the kernel stops after writing
// them to workspace [S][M][N]; bias, activation and residual are then the caller's to apply (lev_linear_mfma_finish, or
// a kernel of its own that reads the ranges).
extern "C" int lev_linear_mfma(const void* a, long lda, const void* w, const float* bias, const float* residual, long ldr,
                               void* out, long ldo, void* workspace, int M, int N, int K, int act, int out_dtype,
                               int leave_ranges, hipStream_t stream) {
  LEV_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
  LEV_REQUIRE(K % 8 == 0 && lda % 8 == 0, "linear (bfloat16): K=%d and the row stride %ld must be multiples of 8", K, lda);
  LEV_REQUIRE(((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0, "linear (bfloat16): operands must be 16-byte aligned");
  LEV_REQUIRE(lda >= K && ldo >= N, "linear: row strides lda=%ld ldo=%ld are smaller than K=%d / N=%d", lda, ldo, K, N);
  LEV_REQUIRE(!residual || (ldr >= N && out_dtype == LEV_F32), "linear: a residual needs a float32 output and a row stride >= N");
  LEV_REQUIRE(act >= LEV_ACT_NONE && act <= LEV_ACT_TANH, "linear: unknown activation %d", act);
  if (M == 0) return 0;
  if (out_dtype == LEV_F32)
    return linear_mfma_typed<float>((const bf16_t*)a, lda, (const bf16_t*)w, bias, residual, ldr, (float*)out, ldo,
                                    (float*)workspace, M, N, K, act, leave_ranges, stream);
  if (out_dtype == LEV_BF16)
    return linear_mfma_typed<bf16_t>((const bf16_t*)a, lda, (const bf16_t*)w, bias, residual, ldr, (bf16_t*)out, ldo,
                                     (float*)workspace, M, N, K, act, leave_ranges, stream);
  return lev_fail("linear: unknown output dtype %d", out_dtype);
}
