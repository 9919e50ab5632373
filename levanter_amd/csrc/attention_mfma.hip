// Causal attention over the paged cache on the matrix cores, bfloat16 in, 32-bit softmax and
// accumulation. Compiled once per head size: -DLEV_HD=<multiple of 16, at most 128>.
//
// Both kernels work on the transposed problem so that no operand needs a transposition:
//   S^T = K . Q^T      A operand: 16 keys x 32 head dims (keys are rows), B operand: Q^T, in registers
//   O^T = V^T . P^T    A operand: 16 head dims x 32 keys from the transposed value pages,
//                      B operand: P^T, which is exactly what the lanes hold after the softmax
// with the 16x16x32 MFMA: A lane l holds row l%16, k = 8*(l/16) .. +7; B lane l holds column l%16,
// the same k; the accumulator's register r of lane l is row 4*(l/16) + r, column l%16.
// The 16 rows of score tile (u, h) (u: which 32 keys of the block of 64, h: which half) are the keys
// 32u + 8*(row/4) + 4h + row%4, so that lane group g = l/16 ends up with the probabilities of the
// 8 consecutive keys 32u + 8g .. +7 in its two tiles: one k-slot run of the second product.
//
// Page layouts (elements): keys [page][kv_head][HD/8][PS][8], values [page][kv_head][HD][PS].
//
//   prefill kernel: one workgroup (8 waves) per (tile of up to 128 consecutive query tokens of one
//                   request, head); keys and values of 64 positions at a time are staged in LDS.
//   decode kernel:  one wave per (single-token query, kv head, split of the key range); operands go
//                   from global memory straight into registers; the splits' partial results
//                   (max, sum, unnormalised output) are merged in a fixed order by a second kernel.
#include "common.h"

#ifndef LEV_HD
#error "compile with -DLEV_HD=<head size>"
#endif

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define HD LEV_HD
#define NCHUNK (HD / 8)            // 16-byte chunks of one key
#define NKS ((HD + 31) / 32)       // k-steps of the score product
#define NDT (HD / 16)              // 16-row tiles of O^T
#define VS_STRIDE 72               // LDS row of V^T: 64 keys + 8 of padding (144 bytes)

#define LEV_CAT_(a, b) a##b
#define LEV_CAT(a, b) LEV_CAT_(a, b)
#define LEV_NAME(base) LEV_CAT(base, LEV_HD)

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) { return float2_to_bf16x2(lo, hi); }
// key (0..63) of row i of score tile (u, h)
__device__ __forceinline__ int tile_key(int u, int h, int i) { return 32 * u + 8 * (i >> 2) + 4 * h + (i & 3); }

// Eight consecutive keys' values of one dimension (two to a word) with all but the first n made zero. A key beyond the
// range has a probability of zero, but what its slot of the cache holds may be anything, NaN too (a page is not cleared
// when it is given to another request), and zero times that would reach the sum.
__device__ __forceinline__ u32x4 first_keys_mask(int n) {
  u32x4 mk;
#pragma unroll
  for (int e = 0; e < 4; ++e) mk[e] = n >= 2 * e + 2 ? 0xffffffffu : (n == 2 * e + 1 ? 0x0000ffffu : 0u);
  return mk;
}

// The largest of the values that lanes l, l ^ 16, l ^ 32 and l ^ 48 hold, in all four of them. The two swaps are vector
// ALU instructions of their own on this chip; the same through ds_bpermute costs two round trips to the LDS, one after the
// other, in the middle of the softmax's chain of dependent steps.
__device__ __forceinline__ float max_over_lane_groups(float v) {
  typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;
  const u32x2_t a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);  // {lower half twice, upper half twice}
  const float w = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const u32x2_t b = __builtin_amdgcn_permlane16_swap(__float_as_uint(w), __float_as_uint(w), false, false);  // {rows 0 0 2 2, rows 1 1 3 3}
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// One block of 64 keys for one wave: scores are in st[u][h] (S^T tiles, raw dot products).
// Applies scale and mask, updates the running max m and sum l (per lane: column = query row),
// rescales the output accumulators and returns the probabilities as B operands pf[u].
// scale_log2 = scale * log2(e): scores, maxima and sums live in the base-2 domain, exp is the bare v_exp_f32.
// q_pos: position of this lane's query row (or -1 for a padding row); key0: position of key 0 of the block.
// need_mask (wave-uniform): false when every key of the block is visible to every row of the tile.
// hook (wave-uniform, off by default): what a model may do to a score between the scaling and the mask
// (src/levanter/layers/attention.py:361-367): add a term that depends on the head and on the distance between query and
// key (bias_row: this lane's head's row of a float32 table [heads][bias_len], distances beyond it take its last entry),
// then cap it softly, cap * tanh(score / cap). Both in natural units, before the change to base 2.
struct ScoreHook {
  float scale;           // the plain scale (scale_log2 / log2(e))
  float softcap;         // 0: none
  const float* bias_row; // null: none
  int bias_len;
};
__device__ __forceinline__ float hooked_score(float raw, const ScoreHook& hk, int q_pos, int kp) {
  float s = raw * hk.scale;
  if (hk.bias_row) s += hk.bias_row[min(max(q_pos - kp, 0), hk.bias_len - 1)];
  if (hk.softcap > 0.f) s = hk.softcap * tanhf(s / hk.softcap);
  return s * 1.4426950408889634f;
}
__device__ __forceinline__ void softmax_block(f32x4 st[2][2], float scale_log2, int q_pos, int lo, int key0, int g,
                                              bool need_mask, float& m, float& l, f32x4* o, u32x4 pf[2], bool hook = false,
                                              const ScoreHook* hk = nullptr) {
  float mx = -INFINITY;
  if (hook) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int kp = key0 + 32 * u + 8 * g + 4 * h + r;
          const bool ok = kp <= q_pos && kp >= lo;
          const float s = ok ? hooked_score(st[u][h][r], *hk, q_pos, kp) : -INFINITY;
          st[u][h][r] = s;
          mx = fmaxf(mx, s);
        }
  } else if (need_mask) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int kp = key0 + 32 * u + 8 * g + 4 * h + r;
          const bool ok = kp <= q_pos && kp >= lo;
          const float s = ok ? st[u][h][r] * scale_log2 : -INFINITY;
          st[u][h][r] = s;
          mx = fmaxf(mx, s);
        }
  } else {
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float s = st[u][h][r] * scale_log2;
          st[u][h][r] = s;
          mx = fmaxf(mx, s);
        }
  }
  mx = max_over_lane_groups(mx);
  const float m_new = fmaxf(m, mx);
  const float base = (m_new == -INFINITY) ? 0.f : m_new;  // a row that has seen no key yet
  const float corr = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - base);
  float psum = 0.f;
  float p[2][2][4];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float e = __builtin_amdgcn_exp2f(st[u][h][r] - base);  // exp2(-inf) = 0 for masked keys
        p[u][h][r] = e;
        psum += e;
      }
  l = l * corr + psum;
  m = m_new;
#pragma unroll
  for (int t = 0; t < NDT; ++t) {
    o[t][0] *= corr; o[t][1] *= corr; o[t][2] *= corr; o[t][3] *= corr;
  }
#pragma unroll
  for (int u = 0; u < 2; ++u)
    pf[u] = u32x4{pack_bf16(p[u][0][0], p[u][0][1]), pack_bf16(p[u][0][2], p[u][0][3]), pack_bf16(p[u][1][0], p[u][1][1]),
                  pack_bf16(p[u][1][2], p[u][1][3])};
}

// The softmax of a block that needs no mask, in two parts so that the products of the next block can be issued between
// them. The running maximum is only raised (and sum and outputs rescaled) when a block's maximum exceeds it by more than
// LAZY_MAX in the base-2 domain: probabilities then reach 2^LAZY_MAX at most, which costs the 32-bit sums nothing, and
// the 4 * NDT multiplications of the rescaling leave nearly every block. m, l and o mean what they mean to softmax_block
// (which takes any m that bounds nothing: it only needs sum and outputs to be scaled by the same exp2(-m)).
#define LAZY_MAX 8.0f
// Part one: is any row's maximum to be raised? (Wave-uniform answer.) m_cand is the lane's candidate.
__device__ __forceinline__ bool softmax_interior_max(const f32x4 st[2][2], float scale_log2, float m, float& m_cand) {
  float mx = fmaxf(fmaxf(st[0][0][0], st[0][0][1]), fmaxf(st[0][0][2], st[0][0][3]));
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int h = 0; h < 2; ++h)
      if (u + h > 0) mx = fmaxf(mx, fmaxf(fmaxf(st[u][h][0], st[u][h][1]), fmaxf(st[u][h][2], st[u][h][3])));
  m_cand = max_over_lane_groups(mx) * scale_log2;  // the scale is positive: the largest raw score is the largest score
  return __builtin_amdgcn_ballot_w64(m_cand > m + LAZY_MAX) != 0;
}
__device__ __forceinline__ void softmax_interior_raise(float m_cand, float& m, float& l, f32x4* o) {
  const float m_new = fmaxf(m, m_cand);
  const float corr = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
  l *= corr;
  m = m_new;
#pragma unroll
  for (int t = 0; t < NDT; ++t) {
    o[t][0] *= corr; o[t][1] *= corr; o[t][2] *= corr; o[t][3] *= corr;
  }
}
// Part two: probabilities (scale and maximum in one multiply-add under the exponential), their sum, and the B operands.
__device__ __forceinline__ void softmax_interior_exp(const f32x4 st[2][2], float scale_log2, float m, float& l, u32x4 pf[2]) {
  float p[2][2][4];
  float psum = 0.f;
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        p[u][h][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[u][h][r], scale_log2, -m));
        psum += p[u][h][r];
      }
  l += psum;
#pragma unroll
  for (int u = 0; u < 2; ++u)
    pf[u] = u32x4{pack_bf16(p[u][0][0], p[u][0][1]), pack_bf16(p[u][0][2], p[u][0][3]), pack_bf16(p[u][1][0], p[u][1][1]),
                  pack_bf16(p[u][1][2], p[u][1][3])};
}

// ------------------------------------------------------------------------------------------------
// Prefill: a workgroup of PF_WAVES waves per (tile of up to PF_ROWS consecutive query tokens, head). Each wave
// owns PF_QT tiles of 16 query rows. Blocks of 64 keys go global -> registers -> LDS, keys and values in two LDS
// buffers each, and the loop is skewed: in the iteration of block kb a wave
//   multiplies the scores of block kb + 1 (matrix pipe, key fragments from LDS),
//   takes the softmax of block kb's scores, which the iteration before left in registers (vector ALU),
//   stages the keys of block kb + 2 and the values of block kb + 1 and requests those after them,
//   multiplies block kb's probabilities with its values (matrix pipe, value fragments from LDS).
// The two products of a block no longer wait for its softmax between them, so that the matrix pipe, the LDS and the
// vector ALU of a wave work at the same time; one barrier an iteration orders the LDS buffers. (With both products and
// the softmax of one block in one iteration, between two barriers, all waves of a CU are in the same phase at the same
// time and each phase waits for another unit: 91 us a layer for a 2,048-token prompt of 32 heads of 128.)
#include "attention_config.h"

typedef bf16_t (*KsPtr)[4][NCHUNK][16][8];  // [buffer][score tile 2u+h][chunk][row][8]
typedef bf16_t (*VsPtr)[HD][VS_STRIDE];     // [buffer][dim][key]

__device__ __forceinline__ void prefill_tile(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long o_stride,
                                             const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                                             const int* __restrict__ positions, const int* __restrict__ token_seq,
                                             const int* __restrict__ block_tables, int bt_stride, int t0, int rows, int h,
                                             int H, int KVH, int ps_shift, float scale, int window, float softcap,
                                             const float* __restrict__ score_bias, int bias_len, KsPtr Ks, VsPtr Vs) {
  if (rows <= 0) return;  // an empty tile (a step filled up to a fixed number of tiles): nothing to do, for the whole workgroup
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int fr = lane & 15, g = lane >> 4;
  const int kvh = h / (H / KVH);
  const float scale_log2 = scale * 1.4426950408889634f;
  const bool hook = softcap > 0.f || score_bias != nullptr;
  const ScoreHook hk = {scale, softcap, score_bias ? score_bias + (size_t)h * bias_len : nullptr, bias_len};
  const int pos0 = positions[t0];
  const int* bt = block_tables + (size_t)token_seq[t0] * bt_stride;
  const int wave_row0 = wave * PF_QT * 16;
  const int hi = pos0 + rows - 1;                                   // last key any row needs
  const int lo_tile = window > 0 ? max(0, pos0 - window + 1) : 0;   // first key any row needs
  int q_pos[PF_QT], lo[PF_QT];
  // Q^T fragments of this lane's query rows, kept for the whole kernel
  u32x4 qf[PF_QT][NKS];
#pragma unroll
  for (int qt = 0; qt < PF_QT; ++qt) {
    const int row = wave_row0 + qt * 16 + fr;
    q_pos[qt] = row < rows ? pos0 + row : -1;
    lo[qt] = window > 0 ? max(0, q_pos[qt] - window + 1) : 0;
#pragma unroll
    for (int s = 0; s < NKS; ++s) {
      const int c = 4 * s + g;
      qf[qt][s] = (q_pos[qt] >= 0 && c < NCHUNK)
                      ? *reinterpret_cast<const u32x4*>(q + (size_t)(t0 + row) * q_stride + (size_t)h * HD + c * 8)
                      : u32x4{0, 0, 0, 0};
    }
  }
  f32x4 o[PF_QT][NDT];
  float m[PF_QT], l[PF_QT];
#pragma unroll
  for (int qt = 0; qt < PF_QT; ++qt) {
    m[qt] = -INFINITY;
    l[qt] = 0.f;
#pragma unroll
    for (int t = 0; t < NDT; ++t) o[qt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // What a thread moves of a block: of K the 16-byte chunks c = wave, wave + PF_WAVES, .. of ONE key (tid % 64); of V
  // 8 consecutive keys of one dimension per chunk. Everything but the page and the block's first key is fixed per thread.
  constexpr int KCH = (64 * NCHUNK + PF_THREADS - 1) / PF_THREADS;  // 16-byte chunks of K per thread and block
  constexpr int VCH = (HD * 8 + PF_THREADS - 1) / PF_THREADS;
  static_assert(PF_THREADS % 64 == 0, "a thread's K chunks belong to one key");
  // Where the chunks of a block are no multiple of the threads, the threads beyond them in the last round repeat the
  // last chunk (the same bytes to the same place): staging has no branch, and the iteration below is one basic block.
  const int ps_mask = (1 << ps_shift) - 1;
  const size_t head_elems = (size_t)HD << ps_shift;
  const size_t page_elems = (size_t)KVH * head_elems;
  const int k_kk = tid & 63;
  size_t k_coff[KCH];
#pragma unroll
  for (int i = 0; i < KCH; ++i) k_coff[i] = (size_t)kvh * head_elems + (((size_t)min((tid >> 6) + PF_WAVES * i, NCHUNK - 1) << ps_shift) * 8);
  int v_kk[VCH];
  size_t v_doff[VCH];
#pragma unroll
  for (int i = 0; i < VCH; ++i) {
    const int y = min(tid + PF_THREADS * i, HD * 8 - 1);
    const int j = y / (HD * 2), rem = y % (HD * 2);
    v_kk[i] = 16 * j + 8 * (rem & 1);  // first of 8 keys; a page holds a multiple of 16
    v_doff[i] = (size_t)kvh * head_elems + ((size_t)(rem >> 1) << ps_shift);
  }
  // Page ids are read an iteration before the data they lead to is requested, so that no data load waits for a table
  // lookup. A key beyond the table's width is beyond `hi` as well and is zeroed when it is staged.
  auto k_page_of = [&](int kb) { return bt[min((kb * 64 + k_kk) >> ps_shift, bt_stride - 1)]; };
  auto v_pages_of = [&](int kb, int page[VCH]) {
#pragma unroll
    for (int i = 0; i < VCH; ++i) page[i] = bt[min((kb * 64 + v_kk[i]) >> ps_shift, bt_stride - 1)];
  };
  u32x4 kr[KCH], vr[VCH];
  // Values beyond the key range are zeroed when they are staged (decided when they are loaded). Keys are staged as they
  // come: a score is looked at only behind the mask, which selects and does not add.
  int vkeep[VCH];  // how many of the chunk's 8 keys are kept
  // Loads are unconditional (a chunk outside the key range reads page 0 and is zeroed when it is staged):
  // conditional loads would make the compiler wait for them at the join instead of after the products.
  auto load_k = [&](int kb, int page) {
    const int kp = kb * 64 + k_kk;
    const bf16_t* base = k_pages + (size_t)max(page, 0) * page_elems + (size_t)(kp & ps_mask) * 8;
#pragma unroll
    for (int i = 0; i < KCH; ++i) kr[i] = *reinterpret_cast<const u32x4*>(base + k_coff[i]);
  };
  auto load_v = [&](int kb, const int page[VCH]) {
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int kp = kb * 64 + v_kk[i];
      vkeep[i] = (kp + 7 >= lo_tile && page[i] >= 0) ? hi - kp + 1 : 0;
      vr[i] = *reinterpret_cast<const u32x4*>(v_pages + (size_t)max(page[i], 0) * page_elems + v_doff[i] + (kp & ps_mask));
    }
  };
  auto stage_k = [&](int buf) {
    const int tile = 2 * (k_kk >> 5) + ((k_kk & 7) >> 2);
    const int row = 4 * ((k_kk & 31) >> 3) + (k_kk & 3);
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = min((tid >> 6) + PF_WAVES * i, NCHUNK - 1);
      *reinterpret_cast<u32x4*>(&Ks[buf][tile][c][row][0]) = kr[i];
    }
  };
  auto stage_v = [&](int buf, bool whole) {  // whole: the block lies in the key range, nothing to zero
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int y = min(tid + PF_THREADS * i, HD * 8 - 1);
      *reinterpret_cast<u32x4*>(&Vs[buf][(y % (HD * 2)) >> 1][v_kk[i]]) = whole ? vr[i] : (vr[i] & first_keys_mask(vkeep[i]));
    }
  };
  const int n_qt = min(PF_QT, max(0, (rows - wave_row0 + 15) / 16));  // query tiles of this wave that hold rows
  // scores of a block for the query tiles that see it (live, wave-uniform), from the keys in Ks[buf]
  auto scores = [&](int buf, const bool live[PF_QT], f32x4 st[PF_QT][2][2]) {
#pragma unroll
    for (int qt = 0; qt < PF_QT; ++qt)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) st[qt][u][hh] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
          const int c = 4 * s + g;
          const u32x4 kf = c < NCHUNK ? *reinterpret_cast<const u32x4*>(&Ks[buf][2 * u + hh][c][fr][0]) : u32x4{0, 0, 0, 0};
#pragma unroll
          for (int qt = 0; qt < PF_QT; ++qt)
            if (live[qt])
              st[qt][u][hh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf), as_bf16x8(qf[qt][s]), st[qt][u][hh], 0, 0, 0);
        }
  };
  auto values = [&](int buf, const bool live[PF_QT], const u32x4 pf[PF_QT][2]) {
#pragma unroll
    for (int t = 0; t < NDT; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const u32x4 vf = *reinterpret_cast<const u32x4*>(&Vs[buf][16 * t + fr][32 * u + 8 * g]);
#pragma unroll
        for (int qt = 0; qt < PF_QT; ++qt)
          if (live[qt]) o[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf), as_bf16x8(pf[qt][u]), o[qt][t], 0, 0, 0);
      }
  };
  auto live_tiles = [&](int kb, bool live[PF_QT]) {  // which query tiles see any key of block kb
    bool any = false;
#pragma unroll
    for (int qt = 0; qt < PF_QT; ++qt) {
      live[qt] = qt < n_qt && kb * 64 <= pos0 + wave_row0 + qt * 16 + 15;
      any = any || live[qt];
    }
    return any;
  };

  const int kb_first = lo_tile / 64, kb_last = hi / 64;
  int kpage, vpage[VCH];
  f32x4 st[PF_QT][2][2];  // raw scores of the block whose softmax comes next
  bool live[PF_QT];
  // Before the loop: K and V of the first block are staged, K of the second, and the scores of the first are taken;
  // K of the third block and V of the second are on their way, the page ids after them are read.
  kpage = k_page_of(kb_first);
  v_pages_of(kb_first, vpage);
  load_k(kb_first, kpage);
  load_v(kb_first, vpage);
  kpage = k_page_of(kb_first + 1);
  v_pages_of(kb_first + 1, vpage);
  lds_barrier();  // a tile before this one (the other of a pair) has been read to its end
  stage_k(0);
  stage_v(0, false);
  load_k(kb_first + 1, kpage);
  load_v(kb_first + 1, vpage);
  kpage = k_page_of(kb_first + 2);
  v_pages_of(kb_first + 2, vpage);
  stage_k(1);
  load_k(kb_first + 2, kpage);
  kpage = k_page_of(kb_first + 3);
  lds_barrier();
  if (live_tiles(kb_first, live)) scores(0, live, st);

  // Iteration of block kb. Ks[cur ^ 1] holds the keys of kb + 1, Vs[cur] the values of kb; kr holds the keys of kb + 2,
  // vr the values of kb + 1 (requested an iteration ago); kpage / vpage are the pages of K(kb + 3) / V(kb + 2).
  auto iteration = [&](int kb, int cur) {
    lds_barrier();  // everyone has staged what this iteration reads and has read what it overwrites
    const int key0 = kb * 64;
    // Every row of the wave sees every key of this block (then it sees some of the next one too) and the values staged
    // now lie in the key range: no branch between the parts of the iteration but the rare one that raises the maxima,
    // and an order of issue given to the compiler. Left alone it emits each part by itself, every product behind a wait
    // for its own LDS read.
    const int p_first = pos0 + wave_row0, p_last = p_first + (PF_QT - 1) * 16 + 15;
    if (!hook && n_qt == PF_QT && key0 + 63 <= p_first && (window <= 0 || p_last - window + 1 <= key0) && key0 + 127 <= hi) {
      bool all[PF_QT];
      float m_cand[PF_QT];
      bool raise = false;
#pragma unroll
      for (int qt = 0; qt < PF_QT; ++qt) {
        all[qt] = true;
        raise = softmax_interior_max(st[qt], scale_log2, m[qt], m_cand[qt]) || raise;
      }
      if (raise) {
#pragma unroll
        for (int qt = 0; qt < PF_QT; ++qt) softmax_interior_raise(m_cand[qt], m[qt], l[qt], o[qt]);
      }
      f32x4 st_next[PF_QT][2][2];
      u32x4 pf[PF_QT][2];
      scores(cur ^ 1, all, st_next);
#pragma unroll
      for (int qt = 0; qt < PF_QT; ++qt) softmax_interior_exp(st[qt], scale_log2, m[qt], l[qt], pf[qt]);
      stage_k(cur);
      stage_v(cur ^ 1, true);
      load_k(kb + 3, kpage);
      load_v(kb + 2, vpage);
      kpage = k_page_of(kb + 4);
      v_pages_of(kb + 3, vpage);
      values(cur, all, pf);
#pragma unroll
      for (int qt = 0; qt < PF_QT; ++qt)
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int hh = 0; hh < 2; ++hh) st[qt][u][hh] = st_next[qt][u][hh];
      // the score products with their key fragments spread over the exponentials ...
      constexpr int N_QK = 4 * NKS * PF_QT, N_KF = 4 * NKS, N_PV = 2 * NDT * PF_QT, N_VF = 2 * NDT;
      constexpr int EXP_VALU = 64 * PF_QT;
      constexpr int AHEAD = 6;  // LDS reads issued before the first product
      __builtin_amdgcn_sched_group_barrier(0x100, AHEAD < N_KF ? AHEAD : N_KF, 0);
#pragma unroll
      for (int i = 0; i < N_QK; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (i * N_KF / N_QK + AHEAD < N_KF && (i * N_KF) % N_QK < N_KF) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, (EXP_VALU + N_QK - 1) / N_QK, 0);
      }
      // ... and the value products with theirs over the staging and the next requests
      __builtin_amdgcn_sched_group_barrier(0x100, AHEAD < N_VF ? AHEAD : N_VF, 0);
#pragma unroll
      for (int i = 0; i < N_PV; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (i * N_VF / N_PV + AHEAD < N_VF && (i * N_VF) % N_PV < N_VF) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        if (i < KCH + VCH) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        else if (i < 2 * (KCH + VCH) + 1 + VCH) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      return;
    }
    bool live_next[PF_QT];
    const bool any = live_tiles(kb, live);
    const bool any_next = kb < kb_last && live_tiles(kb + 1, live_next);
    f32x4 st_next[PF_QT][2][2];
    u32x4 pf[PF_QT][2];
    if (any_next) scores(cur ^ 1, live_next, st_next);
    if (any) {
#pragma unroll
      for (int qt = 0; qt < PF_QT; ++qt)
        if (live[qt]) {
          const int p0 = pos0 + wave_row0 + qt * 16;  // first row of the tile: does it see the whole block, and the last row too
          const bool need_mask = !(key0 + 63 <= p0 && (window <= 0 || p0 + 15 - window + 1 <= key0));
          softmax_block(st[qt], scale_log2, q_pos[qt], lo[qt], key0, g, need_mask, m[qt], l[qt], o[qt], pf[qt], hook, &hk);
        }
    }
    stage_k(cur);              // K(kb + 2) over K(kb), which the iteration before read
    stage_v(cur ^ 1, false);   // V(kb + 1) over V(kb - 1)
    load_k(kb + 3, kpage);  // blocks past the last one are zeroed by their key positions
    load_v(kb + 2, vpage);
    kpage = k_page_of(kb + 4);
    v_pages_of(kb + 3, vpage);
    if (any) values(cur, live, pf);
    if (any_next) {
#pragma unroll
      for (int qt = 0; qt < PF_QT; ++qt)
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int hh = 0; hh < 2; ++hh) st[qt][u][hh] = st_next[qt][u][hh];
    }
  };
  int kb = kb_first;
  for (; kb + 1 <= kb_last; kb += 2) {
    iteration(kb, 0);
    iteration(kb + 1, 1);
  }
  if (kb <= kb_last) iteration(kb, 0);
#pragma unroll
  for (int qt = 0; qt < PF_QT; ++qt) {
    float lq = l[qt];
    lq += __shfl_xor(lq, 16, 64);
    lq += __shfl_xor(lq, 32, 64);
    if (q_pos[qt] >= 0) {
      const float inv = 1.0f / lq;
      bf16_t* orow = out + (size_t)(t0 + wave_row0 + qt * 16 + fr) * o_stride + (size_t)h * HD;
#pragma unroll
      for (int t = 0; t < NDT; ++t) {
        const u32x2 v = u32x2{pack_bf16(o[qt][t][0] * inv, o[qt][t][1] * inv), pack_bf16(o[qt][t][2] * inv, o[qt][t][3] * inv)};
        *reinterpret_cast<u32x2*>(orow + 16 * t + 4 * g) = v;
      }
    }
  }
}

// Workgroup b of n (n = H times the number of tiles, or of pairs of tiles): its tile (or pair) x and its head h.
__device__ __forceinline__ void prefill_workgroup(int b, int n, int H, int KVH, int& x, int& h) {
  const int n_x = n / H;
  if (KVH % 8 == 0) {
    const int xcd = b % 8, j = b / 8, G = H / KVH;
    const int kvh = xcd + 8 * (j % (KVH / 8)), rest = j / (KVH / 8);  // rest counts (query head of the group, tile)
    h = kvh * G + rest % G;
    x = rest / G;
  } else {
    x = b % n_x;
    h = b / n_x;
  }
}

// The tiles come sorted by falling number of key blocks; with `pair`, workgroup x takes tile x and then tile n - 1 - x,
// so that every workgroup has about the same work (a causal prompt's last tile reads many times more keys than its first).
__global__ void __launch_bounds__(PF_THREADS)
LEV_NAME(attn_prefill_hd)(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long o_stride,
                          const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                          const int* __restrict__ positions, const int* __restrict__ token_seq,
                          const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ tiles, int n_tiles, int pair,
                          int H, int KVH, int ps_shift, float scale, int window, float softcap,
                          const float* __restrict__ score_bias, int bias_len) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[2][4][NCHUNK][16][8];  // [buffer][score tile 2u+h][chunk][row][8]
  __shared__ __attribute__((aligned(16))) bf16_t Vs[2][HD][VS_STRIDE];
  // Workgroups go to the 8 XCDs in turn, each with an L2 of its own. A kv head's keys and values are read by every tile
  // of every query head that shares it: all of those run on one XCD (kv head % 8), so that the cache is fetched from
  // memory about once and not once per XCD (a 2,048-token prompt of 32 heads of 128: 34 MB a layer against 285 MB).
  int x, h;
  prefill_workgroup(blockIdx.x, gridDim.x, H, KVH, x, h);
  const int first = x, second = n_tiles - 1 - x;
  prefill_tile(q, q_stride, out, o_stride, k_pages, v_pages, positions, token_seq, block_tables, bt_stride, tiles[2 * first],
               tiles[2 * first + 1], h, H, KVH, ps_shift, scale, window, softcap, score_bias, bias_len, Ks, Vs);
  if (pair && second > first)
    prefill_tile(q, q_stride, out, o_stride, k_pages, v_pages, positions, token_seq, block_tables, bt_stride, tiles[2 * second],
                 tiles[2 * second + 1], h, H, KVH, ps_shift, scale, window, softcap, score_bias, bias_len, Ks, Vs);
}

// ------------------------------------------------------------------------------------------------
// Decode: one wave per (token, kv head, split). Columns of Q^T are the G = H / KVH query heads that
// share the kv head. With more than one split the partial results are merged in the order of the splits:
//   wg_merge: the splits of a (token, kv head) are the waves of ONE workgroup (up to DECODE_WG_WAVES); they leave
//     m, l and o in LDS and, behind a barrier, the workgroup's threads merge them and write the output;
//   else (more splits than that, or too many query heads per kv head for the LDS): one workgroup per split,
//     partial results in the workspace  ws_m, ws_l [token][head][split], ws_o [token][head][split][HD],  and a
//     second kernel merges them. (Merging in the last workgroup to finish, behind an atomic ticket, was measured:
//     the device-scope fences it needs cost several times the second launch.)
//
// k_new != null: the step's new key and value of each token are not in the cache yet. The wave whose key
// range holds the token's own position takes them from k_new / v_new (rows of the projection's output) and
// uses them in place of what the cache holds there; one wave copies them to dest[t] = page * PS + offset.
#define DECODE_WG_WAVES 8
// One wave's work: single token number idx of the step, kv head kvh, key range z of `splits`.
__device__ __forceinline__ void decode_wave(int idx, int kvh, int z, const bf16_t* __restrict__ q, long q_stride,
                                            bf16_t* __restrict__ out, long o_stride, bf16_t* __restrict__ k_pages,
                                            bf16_t* __restrict__ v_pages, const int* __restrict__ positions,
                                            const int* __restrict__ token_seq, const int* __restrict__ block_tables, int bt_stride,
                                            const int* __restrict__ decode_tokens, const bf16_t* __restrict__ k_new,
                                            const bf16_t* __restrict__ v_new, long kv_stride, const int* __restrict__ dest,
                                            float* __restrict__ ws_m, float* __restrict__ ws_l, float* __restrict__ ws_o, int H,
                                            int KVH, int ps_shift, int splits, float scale, int window, int wg_merge, float softcap,
                                            const float* __restrict__ score_bias, int bias_len) {
  const int PS = 1 << ps_shift, ps_mask = PS - 1;
  const float scale_log2 = scale * 1.4426950408889634f;
  const int lane = threadIdx.x & 63;
  const int fr = lane & 15, g = lane >> 4;
  const int t = decode_tokens[idx];
  const int G = H / KVH;
  const int pos = positions[t];
  const int* bt = block_tables + (size_t)token_seq[t] * bt_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int kb_first = lo / 64, kb_last = pos / 64;
  const int per = (kb_last - kb_first + 1 + splits - 1) / splits;
  const int kb_begin = kb_first + z * per, kb_end = min(kb_last + 1, kb_begin + per);
  const int head = kvh * G + fr;  // this lane's query head (column of Q^T)
  const int q_pos = fr < G ? pos : -1;
  const bool hook = softcap > 0.f || score_bias != nullptr;
  const ScoreHook hk = {scale, softcap, score_bias ? score_bias + (size_t)min(head, H - 1) * bias_len : nullptr, bias_len};
  const size_t head_elems = (size_t)HD << ps_shift;
  const bool fused = k_new != nullptr;
  // The new key and value are copied to their page by one wave of the (token, kv head): the last one if it has no keys
  // of its own (the ranges are rounded up, so with few blocks the last waves are idle), else the wave whose range
  // holds the token's position, which then has the copy ahead of its two or more blocks.
  const bool idle_last = splits > 1 && kb_first + (splits - 1) * per > kb_last;
  const bool owner = fused && (idle_last ? z == splits - 1 : (kb_begin <= kb_last && kb_last < kb_end));
  const bf16_t* kn = fused ? k_new + (size_t)t * kv_stride + (size_t)kvh * HD : nullptr;
  const bf16_t* vn = fused ? v_new + (size_t)t * kv_stride + (size_t)kvh * HD : nullptr;

  if (owner) {  // read by later steps only: this step takes them from k_new / v_new
    const int dst = dest[t];
    if (dst >= 0) {
      bf16_t* kb_ = k_pages + ((size_t)(dst >> ps_shift) * KVH + kvh) * head_elems;
      bf16_t* vb_ = v_pages + ((size_t)(dst >> ps_shift) * KVH + kvh) * head_elems;
      const int off = dst & ps_mask;
      for (int c = lane; c < NCHUNK; c += 64)
        *reinterpret_cast<u32x4*>(kb_ + ((size_t)c * PS + off) * 8) = *reinterpret_cast<const u32x4*>(kn + c * 8);
      for (int d = lane; d < HD; d += 64) vb_[(size_t)d * PS + off] = vn[d];
    }
  }

  u32x4 qf[NKS];
#pragma unroll
  for (int s = 0; s < NKS; ++s) {
    const int c = 4 * s + g;
    qf[s] = (q_pos >= 0 && c < NCHUNK) ? *reinterpret_cast<const u32x4*>(q + (size_t)t * q_stride + (size_t)head * HD + c * 8)
                                        : u32x4{0, 0, 0, 0};
  }
  f32x4 o[NDT];
#pragma unroll
  for (int i = 0; i < NDT; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // Every load below is unconditional, from a clamped address, and what it must not deliver is masked out afterwards:
  // a load under a condition becomes a branch, and at the join the compiler waits for all loads in flight, which
  // turned the 38 loads of a block into as many round trips to memory, one after the other.
  // This lane's rows of the token's new value, read once, two to a register.
  uint32_t nv2[(NDT + 1) / 2];
#pragma unroll
  for (int i = 0; i < (NDT + 1) / 2; ++i) nv2[i] = 0u;
  if (fused) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) nv2[dt / 2] |= (uint32_t)vn[16 * dt + fr] << (16 * (dt & 1));
  }
  // Page ids of a block of 64 keys, per lane: one per key tile (u, hh) and one per group of 8 values (u). They are read
  // one block ahead (behind the block's own loads, into the registers those have just used), so that no key or value
  // load waits for a table lookup. Positions beyond the token's own are clamped to it (its table entry exists);
  // vector loads on purpose (the index is made opaque).
  int kpg[2][2], vpg[2];
  auto page_ids = [&](int kb) {
    const int key0 = kb * 64;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        int at = min(key0 + tile_key(u, hh, fr), pos) >> ps_shift;
        asm volatile("" : "+v"(at));
        kpg[u][hh] = bt[at];
      }
      int at = min(key0 + 32 * u + 8 * g, pos) >> ps_shift;
      asm volatile("" : "+v"(at));
      vpg[u] = bt[at];
    }
  };
  page_ids(min(kb_begin, kb_last));
  for (int kb = kb_begin; kb < kb_end; ++kb) {
    const int key0 = kb * 64;
    // key operands: tile (u, hh), row fr is key tile_key(u, hh, fr)
    u32x4 kf[2][2][NKS];
    uint32_t k_mask[2][2];  // all ones where the key is in the range
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int kp = key0 + tile_key(u, hh, fr);
        const bool is_new = fused && kp == pos;
        const int page = kpg[u][hh];
        k_mask[u][hh] = (kp <= pos && kp >= lo && (page >= 0 || is_new)) ? 0xffffffffu : 0u;
        const bf16_t* base = is_new ? kn : k_pages + ((size_t)max(page, 0) * KVH + kvh) * head_elems + (size_t)(kp & ps_mask) * 8;
        const size_t cstride = is_new ? 8 : (size_t)PS * 8;
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
          const int c = min(4 * s + g, NCHUNK - 1);
          kf[u][hh][s] = *reinterpret_cast<const u32x4*>(base + (size_t)c * cstride);
        }
      }
    // value operands: tile dt, row fr is head dim 16*dt + fr, k-slots are keys 32u + 8g .. +7
    u32x4 vf[NDT][2];
    u32x4 v_mask[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kp = key0 + 32 * u + 8 * g;
      const int page = vpg[u];
      v_mask[u] = first_keys_mask((kp + 7 >= lo && page >= 0) ? pos - kp + 1 : 0);
      const bf16_t* base = v_pages + ((size_t)max(page, 0) * KVH + kvh) * head_elems + (kp & ps_mask);
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) vf[dt][u] = *reinterpret_cast<const u32x4*>(base + (size_t)(16 * dt + fr) * PS);
    }
    page_ids(kb + 1);
    // what the loads must not deliver: keys outside the range and chunks beyond the head size become zero
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
          const uint32_t mk = 4 * s + g < NCHUNK ? k_mask[u][hh] : 0u;
          kf[u][hh][s] = kf[u][hh][s] & u32x4{mk, mk, mk, mk};
        }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int jn = pos - (key0 + 32 * u + 8 * g);  // slot of the new value among this lane's 8 keys, if 0 <= jn < 8
      const bool has_new = fused && jn >= 0 && jn < 8;
      const int w = jn >> 1;
      // the new value replaces one half of word w: keep-mask and shift of that half
      const uint32_t keep = (jn & 1) ? 0x0000ffffu : 0xffff0000u;
      const int shift = (jn & 1) ? 16 : 0;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        u32x4 v = vf[dt][u] & v_mask[u];
        const uint32_t nvd = (nv2[dt / 2] >> (16 * (dt & 1))) & 0xffffu;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (has_new && w == e) ? ((v[e] & keep) | (nvd << shift)) : v[e];
        vf[dt][u] = v;
      }
    }
    f32x4 st[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NKS; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf[u][hh][s]), as_bf16x8(qf[s]), acc, 0, 0, 0);
        st[u][hh] = acc;
      }
    u32x4 pf[2];
    softmax_block(st, scale_log2, q_pos, lo, key0, g, key0 + 63 > pos || key0 < lo, m, l, o, pf, hook, &hk);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int u = 0; u < 2; ++u)
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf[dt][u]), as_bf16x8(pf[u]), o[dt], 0, 0, 0);
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (splits == 1) {
    if (q_pos >= 0) {
      const float inv = 1.0f / l;
      bf16_t* orow = out + (size_t)t * o_stride + (size_t)head * HD;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        const u32x2 v = u32x2{pack_bf16(o[dt][0] * inv, o[dt][1] * inv), pack_bf16(o[dt][2] * inv, o[dt][3] * inv)};
        *reinterpret_cast<u32x2*>(orow + 16 * dt + 4 * g) = v;
      }
    }
    return;
  }
  if (wg_merge) {
    // partial results of this wave into LDS [split][query head of the group]: m, l, o[HD]
    extern __shared__ float merge_s[];
    float* ms = merge_s;
    float* ls = ms + splits * G;
    float* os = ls + splits * G;
    if (fr < G) {
      if (g == 0) {
        ms[z * G + fr] = m;
        ls[z * G + fr] = l;
      }
      float* wo = os + (size_t)(z * G + fr) * HD;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f32x4*>(wo + 16 * dt + 4 * g) = o[dt];
    }
    __syncthreads();
    bf16_t* orow = out + (size_t)t * o_stride + (size_t)kvh * G * HD;
    for (int e = threadIdx.x; e < G * HD; e += blockDim.x) {
      const int hq = e / HD, d = e - hq * HD;
      float mx = -INFINITY;
      for (int zz = 0; zz < splits; ++zz) mx = fmaxf(mx, ms[zz * G + hq]);
      float lsum = 0.f, acc = 0.f;
      for (int zz = 0; zz < splits; ++zz) {  // the maxima are in the base-2 domain
        const float mz = ms[zz * G + hq];
        const float wz = mz == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mz - mx);
        lsum += ls[zz * G + hq] * wz;
        acc += os[(size_t)(zz * G + hq) * HD + d] * wz;
      }
      orow[(size_t)hq * HD + d] = float_to_bf16(acc / lsum);
    }
    return;
  }
  if (q_pos >= 0) {
    const size_t slot = ((size_t)idx * H + head) * splits + z;
    if (g == 0) {
      ws_m[slot] = m;
      ws_l[slot] = l;
    }
    float* wo = ws_o + slot * HD;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f32x4*>(wo + 16 * dt + 4 * g) = o[dt];
  }
}

__global__ void __launch_bounds__(64 * DECODE_WG_WAVES)
LEV_NAME(attn_decode_hd)(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long o_stride,
                         bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, const int* __restrict__ positions,
                         const int* __restrict__ token_seq, const int* __restrict__ block_tables, int bt_stride,
                         const int* __restrict__ decode_tokens, const bf16_t* __restrict__ k_new,
                         const bf16_t* __restrict__ v_new, long kv_stride, const int* __restrict__ dest,
                         float* __restrict__ ws_m, float* __restrict__ ws_l, float* __restrict__ ws_o,
                         int H, int KVH, int ps_shift, int splits, float scale, int window, int wg_merge, float softcap,
                         const float* __restrict__ score_bias, int bias_len) {
  decode_wave(blockIdx.x, blockIdx.y, wg_merge ? (int)(threadIdx.x >> 6) : (int)blockIdx.z, q, q_stride, out, o_stride, k_pages, v_pages,
              positions, token_seq, block_tables, bt_stride, decode_tokens, k_new, v_new, kv_stride, dest, ws_m, ws_l, ws_o, H, KVH,
              ps_shift, splits, scale, window, wg_merge, softcap, score_bias, bias_len);
}

// A step of prompt portions beside single tokens whose key ranges are not split: both kinds of work in one launch, so that
// the single tokens' waves (bound by memory) fill the CUs that the portions' few workgroups (bound by latency) leave idle,
// and the step has one kernel boundary fewer a layer. Workgroups below n_pf_wgs are the prefill kernel's, with its
// numbering; each of the others is DECODE_WG_WAVES waves with a (single token, kv head) each, whose new keys and values
// the KV-write kernel has written before.
__global__ void __launch_bounds__(PF_THREADS)
LEV_NAME(attn_mixed_hd)(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long o_stride,
                        bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, const int* __restrict__ positions,
                        const int* __restrict__ token_seq, const int* __restrict__ block_tables, int bt_stride,
                        const int* __restrict__ tiles, int n_tiles, int pair, int n_pf_wgs, const int* __restrict__ decode_tokens,
                        int n_decode, int H, int KVH, int ps_shift, float scale, int window, float softcap,
                        const float* __restrict__ score_bias, int bias_len) {
  static_assert(PF_THREADS == 64 * DECODE_WG_WAVES, "one workgroup size for both kinds of work");
  __shared__ __attribute__((aligned(16))) bf16_t Ks[2][4][NCHUNK][16][8];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[2][HD][VS_STRIDE];
  if ((int)blockIdx.x < n_pf_wgs) {
    int x, h;
    prefill_workgroup(blockIdx.x, n_pf_wgs, H, KVH, x, h);
    const int first = x, second = n_tiles - 1 - x;
    prefill_tile(q, q_stride, out, o_stride, k_pages, v_pages, positions, token_seq, block_tables, bt_stride, tiles[2 * first],
                 tiles[2 * first + 1], h, H, KVH, ps_shift, scale, window, softcap, score_bias, bias_len, Ks, Vs);
    if (pair && second > first)
      prefill_tile(q, q_stride, out, o_stride, k_pages, v_pages, positions, token_seq, block_tables, bt_stride, tiles[2 * second],
                   tiles[2 * second + 1], h, H, KVH, ps_shift, scale, window, softcap, score_bias, bias_len, Ks, Vs);
    return;
  }
  const int item = ((int)blockIdx.x - n_pf_wgs) * DECODE_WG_WAVES + (int)(threadIdx.x >> 6);
  if (item >= n_decode * KVH) return;
  decode_wave(item / KVH, item % KVH, 0, q, q_stride, out, o_stride, k_pages, v_pages, positions, token_seq, block_tables, bt_stride,
              decode_tokens, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, H, KVH, ps_shift, 1, scale, window, 0, softcap,
              score_bias, bias_len);
}

// merge the splits of one (token, head): weights exp(m_z - max) per split, then a fixed-order sum
__global__ void __launch_bounds__(64)
LEV_NAME(attn_combine_hd)(bf16_t* __restrict__ out, long o_stride, const int* __restrict__ decode_tokens,
                          const float* __restrict__ ws_m, const float* __restrict__ ws_l, const float* __restrict__ ws_o,
                          int H, int splits) {
  __shared__ float wz[64];
  const int idx = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const size_t slot0 = ((size_t)idx * H + head) * splits;
  const float mz = lane < splits ? ws_m[slot0 + lane] : -INFINITY;
  const float lz = lane < splits ? ws_l[slot0 + lane] : 0.f;
  const float mx = wave_max(mz);
  const float w = mz == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mz - mx);  // the maxima are in the base-2 domain
  wz[lane] = w;
  const float l = wave_sum(lz * w);  // summed over the lanes in a fixed butterfly order
  __syncthreads();
  const float inv = 1.0f / l;
  bf16_t* orow = out + (size_t)decode_tokens[idx] * o_stride + (size_t)head * HD;
  for (int d = lane; d < HD; d += 64) {
    float acc = 0.f;
    int z = 0;
    for (; z + 4 <= splits; z += 4) {
      const float a0 = ws_o[(slot0 + z) * HD + d], a1 = ws_o[(slot0 + z + 1) * HD + d];
      const float a2 = ws_o[(slot0 + z + 2) * HD + d], a3 = ws_o[(slot0 + z + 3) * HD + d];
      acc += a0 * wz[z];
      acc += a1 * wz[z + 1];
      acc += a2 * wz[z + 2];
      acc += a3 * wz[z + 3];
    }
    for (; z < splits; ++z) acc += ws_o[(slot0 + z) * HD + d] * wz[z];
    orow[d] = float_to_bf16(acc * inv);
  }
}

extern "C" int LEV_NAME(lev_attention_mfma_hd)(const void* q, long q_stride, void* out, long o_stride, void* k_pages,
                                               void* v_pages, const int* positions, const int* token_seq,
                                               const int* block_tables, int bt_stride, const int* prefill_tiles,
                                               int n_prefill_tiles, const int* decode_tokens, int n_decode, const void* k_new,
                                               const void* v_new, long kv_stride, const int* dest, void* workspace, int H,
                                               int KVH, int PS, int splits, float scale, int window, float softcap,
                                               const float* score_bias, int bias_len, hipStream_t stream) {
  int ps_shift = 0;
  while ((1 << ps_shift) < PS) ++ps_shift;
  if ((1 << ps_shift) != PS) return lev_fail("attention (matrix cores): page_size=%d must be a power of two", PS);
  if (n_prefill_tiles > 0 && n_decode > 0 && splits == 1 && !k_new) {
    const int pair = (long)n_prefill_tiles * H >= 512;
    const int n_pf_wgs = (pair ? (n_prefill_tiles + 1) / 2 : n_prefill_tiles) * H;
    const long items = (long)n_decode * KVH;
    dim3 grid((unsigned)(n_pf_wgs + (items + DECODE_WG_WAVES - 1) / DECODE_WG_WAVES));
    LEV_NAME(attn_mixed_hd)<<<grid, PF_THREADS, 0, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, o_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, positions, token_seq, block_tables,
        bt_stride, prefill_tiles, n_prefill_tiles, pair, n_pf_wgs, decode_tokens, n_decode, H, KVH, ps_shift, scale, window, softcap,
        score_bias, bias_len);
    return lev_check_launch("attention of a mixed step");
  }
  if (n_prefill_tiles > 0) {
    // pairing halves the number of workgroups: only when every CU (256 of them) still gets one
    const int pair = (long)n_prefill_tiles * H >= 512;
    dim3 grid((pair ? (n_prefill_tiles + 1) / 2 : n_prefill_tiles) * H);
    LEV_NAME(attn_prefill_hd)<<<grid, PF_THREADS, 0, stream>>>((const bf16_t*)q, q_stride, (bf16_t*)out, o_stride,
                                                        (const bf16_t*)k_pages, (const bf16_t*)v_pages, positions, token_seq,
                                                        block_tables, bt_stride, prefill_tiles, n_prefill_tiles, pair, H,
                                                        KVH, ps_shift, scale, window, softcap, score_bias, bias_len);
    if (int rc = lev_check_launch("attention prefill")) return rc;
  }
  if (n_decode > 0) {
    // workspace: m, l, o of every (token, head, split)
    const size_t rows = (size_t)n_decode * H * splits;
    float* ws_m = (float*)workspace;
    float* ws_l = ws_m + rows;
    float* ws_o = ws_l + rows;
    const int G = H / KVH;
    const size_t merge_bytes = (size_t)splits * G * (HD + 2) * sizeof(float);
    const int wg_merge = splits > 1 && splits <= DECODE_WG_WAVES && merge_bytes <= 48 * 1024;
    dim3 grid(n_decode, KVH, wg_merge ? 1 : splits);
    LEV_NAME(attn_decode_hd)<<<grid, wg_merge ? 64 * splits : 64, wg_merge ? merge_bytes : 0, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, o_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, positions, token_seq, block_tables,
        bt_stride, decode_tokens, (const bf16_t*)k_new, (const bf16_t*)v_new, kv_stride, dest, ws_m, ws_l, ws_o, H, KVH, ps_shift,
        splits, scale, window, wg_merge, softcap, score_bias, bias_len);
    if (int rc = lev_check_launch("attention decode")) return rc;
    if (splits > 1 && !wg_merge) {
      dim3 cgrid(n_decode, H);
      LEV_NAME(attn_combine_hd)<<<cgrid, 64, 0, stream>>>((bf16_t*)out, o_stride, decode_tokens, ws_m, ws_l, ws_o, H, splits);
      if (int rc = lev_check_launch("attention combine")) return rc;
    }
  }
  return 0;
}
