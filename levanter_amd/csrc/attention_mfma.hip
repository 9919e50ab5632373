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
//   prefill kernel: one workgroup (4 waves) per (tile of up to 64 consecutive query tokens of one
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

// One block of 64 keys for one wave: scores are in st[u][h] (S^T tiles, raw dot products).
// Applies scale and mask, updates the running max m and sum l (per lane: column = query row),
// rescales the output accumulators and returns the probabilities as B operands pf[u].
// scale_log2 = scale * log2(e): scores, maxima and sums live in the base-2 domain, exp is the bare v_exp_f32.
// q_pos: position of this lane's query row (or -1 for a padding row); key0: position of key 0 of the block.
// need_mask (wave-uniform): false when every key of the block is visible to every row of the tile.
__device__ __forceinline__ void softmax_block(f32x4 st[2][2], float scale_log2, int q_pos, int lo, int key0, int g,
                                              bool need_mask, float& m, float& l, f32x4* o, u32x4 pf[2]) {
  float mx = -INFINITY;
  if (need_mask) {
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
  mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
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

// ------------------------------------------------------------------------------------------------
// Prefill: a workgroup of PF_WAVES waves per (tile of up to PF_ROWS consecutive query tokens, head). Each wave
// owns PF_QT tiles of 16 query rows: a key or value fragment read from LDS feeds PF_QT products, which is what
// keeps the kernel off the LDS bandwidth limit. Blocks of 64 keys go global -> registers -> LDS; the loads of
// the next block are in flight during the products (barriers order LDS only).
#include "attention_config.h"

typedef bf16_t (*KsPtr)[NCHUNK][16][8];
typedef bf16_t (*VsPtr)[VS_STRIDE];

__device__ __forceinline__ void prefill_tile(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long o_stride,
                                             const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                                             const int* __restrict__ positions, const int* __restrict__ token_seq,
                                             const int* __restrict__ block_tables, int bt_stride, int t0, int rows, int h,
                                             int H, int KVH, int ps_shift, float scale, int window, KsPtr Ks, VsPtr Vs) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int fr = lane & 15, g = lane >> 4;
  const int kvh = h / (H / KVH);
  const float scale_log2 = scale * 1.4426950408889634f;
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

  constexpr int KCH = (64 * NCHUNK + PF_THREADS - 1) / PF_THREADS;  // 16-byte chunks of K per thread and block
  constexpr int VCH = (HD * 8 + PF_THREADS - 1) / PF_THREADS;
  // two register sets: block kb + 2 is loaded while block kb is multiplied (a load has two iterations to arrive)
  u32x4 kr[2][KCH], vr[2][VCH];
  bool kok[2][KCH], vok[2][VCH];  // does the chunk hold keys of the range (decided when it is loaded, used when it is staged)
  const int PS = 1 << ps_shift, ps_mask = PS - 1;
  const size_t head_elems = (size_t)HD << ps_shift;
  // The page ids of a block of 64 keys (at most 4 of them) are read one iteration before the block's data is
  // requested, so that no data load waits for a table lookup. They are read with vector loads on purpose (the
  // index is made opaque): scalar loads share a counter with LDS and, while one is in flight, the compiler
  // waits for every LDS read at once instead of pipelining them.
  constexpr int NPG = 4;
  // pg[0..3]: the ids as loaded (not looked at until the next iteration, so nothing waits for the loads here);
  // pg[4]: bit j says whether entry j exists
  auto load_pages = [&](int kb, int pg[NPG + 1]) {
    const int b0 = (kb * 64) >> ps_shift;
    int valid = 0;
#pragma unroll
    for (int j = 0; j < NPG; ++j) {
      const int idx = b0 + j;
      int at = min(idx, bt_stride - 1);
      asm volatile("" : "+v"(at));
      pg[j] = bt[at];
      valid |= (idx < bt_stride && (j << ps_shift) < 64) ? (1 << j) : 0;
    }
    pg[NPG] = valid;
  };
  auto pick = [&](const int pg[NPG + 1], int j) {
    const int v = j == 0 ? pg[0] : (j == 1 ? pg[1] : (j == 2 ? pg[2] : pg[3]));
    return ((pg[NPG] >> j) & 1) ? v : -1;
  };
  // Loads are unconditional (a chunk outside the key range reads page 0 and is zeroed when it is staged):
  // conditional loads would make the compiler wait for them at the join instead of after the products.
  auto prefetch = [&](int set, int kb, const int pg[NPG + 1]) {
    const int key0 = kb * 64;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int x = tid + PF_THREADS * i;
      const int kk = x & 63, c = min(x >> 6, NCHUNK - 1);
      const int kp = key0 + kk;
      const int page = pick(pg, kk >> ps_shift);
      kok[set][i] = kp <= hi && kp >= lo_tile && page >= 0;
      kr[set][i] = *reinterpret_cast<const u32x4*>(k_pages + ((size_t)max(page, 0) * KVH + kvh) * head_elems + (((size_t)c << ps_shift) + (kp & ps_mask)) * 8);
    }
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int y = min(tid + PF_THREADS * i, HD * 8 - 1);
      const int j = y / (HD * 2), rem = y % (HD * 2);
      const int d = rem >> 1, half = rem & 1;
      const int kk = 16 * j + 8 * half;  // first of 8 keys; a page holds a multiple of 16
      const int kp = key0 + kk;
      const int page = pick(pg, kk >> ps_shift);
      vok[set][i] = kp <= hi && kp + 7 >= lo_tile && page >= 0;
      vr[set][i] = *reinterpret_cast<const u32x4*>(v_pages + ((size_t)max(page, 0) * KVH + kvh) * head_elems + ((size_t)d << ps_shift) + (kp & ps_mask));
    }
  };
  auto stage = [&](int set) {
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int x = tid + PF_THREADS * i;
      const int kk = x & 63, c = x >> 6;
      if (c < NCHUNK) {
        const int tile = 2 * (kk >> 5) + ((kk & 7) >> 2);
        const int row = 4 * ((kk & 31) >> 3) + (kk & 3);
        *reinterpret_cast<u32x4*>(&Ks[tile][c][row][0]) = kok[set][i] ? kr[set][i] : u32x4{0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int y = tid + PF_THREADS * i;
      if (y < HD * 8) {
        const int j = y / (HD * 2), rem = y % (HD * 2);
        *reinterpret_cast<u32x4*>(&Vs[rem >> 1][16 * j + 8 * (rem & 1)]) = vok[set][i] ? vr[set][i] : u32x4{0, 0, 0, 0};
      }
    }
  };

  const int kb_first = lo_tile / 64, kb_last = hi / 64;
  const int n_qt = min(PF_QT, max(0, (rows - wave_row0 + 15) / 16));  // query tiles of this wave that hold rows
  int pgs[2][NPG + 1];  // page ids of the blocks with even / odd distance from the first
  load_pages(kb_first, pgs[0]);
  load_pages(kb_first + 1, pgs[1]);
  prefetch(0, kb_first, pgs[0]);
  prefetch(1, kb_first + 1, pgs[1]);
  load_pages(kb_first + 2, pgs[0]);
  auto block = [&](int kb, int set) {
    lds_barrier();  // everyone has finished reading the previous block
    stage(set);
    lds_barrier();
    load_pages(kb + 3, pgs[set ^ 1]);  // older than the data loads below: waiting for them later leaves those in flight
    prefetch(set, kb + 2, pgs[set]);   // blocks past the last one are masked by their key positions
    const int key0 = kb * 64;
    bool live[PF_QT];  // does query tile qt see any key of this block (wave-uniform)
    bool any = false;
#pragma unroll
    for (int qt = 0; qt < PF_QT; ++qt) {
      live[qt] = qt < n_qt && key0 <= pos0 + wave_row0 + qt * 16 + 15;
      any = any || live[qt];
    }
    if (!any) return;
    f32x4 st[PF_QT][2][2];
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
          const u32x4 kf = c < NCHUNK ? *reinterpret_cast<const u32x4*>(&Ks[2 * u + hh][c][fr][0]) : u32x4{0, 0, 0, 0};
#pragma unroll
          for (int qt = 0; qt < PF_QT; ++qt)
            if (live[qt])
              st[qt][u][hh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf), as_bf16x8(qf[qt][s]), st[qt][u][hh], 0, 0, 0);
        }
    u32x4 pf[PF_QT][2];
#pragma unroll
    for (int qt = 0; qt < PF_QT; ++qt)
      if (live[qt]) {
        const int p0 = pos0 + wave_row0 + qt * 16;  // first row of the tile: does it see the whole block, and the last row too
        const bool need_mask = !(key0 + 63 <= p0 && (window <= 0 || p0 + 15 - window + 1 <= key0));
        softmax_block(st[qt], scale_log2, q_pos[qt], lo[qt], key0, g, need_mask, m[qt], l[qt], o[qt], pf[qt]);
      }
#pragma unroll
    for (int t = 0; t < NDT; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const u32x4 vf = *reinterpret_cast<const u32x4*>(&Vs[16 * t + fr][32 * u + 8 * g]);
#pragma unroll
        for (int qt = 0; qt < PF_QT; ++qt)
          if (live[qt]) o[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf), as_bf16x8(pf[qt][u]), o[qt][t], 0, 0, 0);
      }
  };
  int kb = kb_first;
  for (; kb + 1 <= kb_last; kb += 2) {
    block(kb, 0);
    block(kb + 1, 1);
  }
  if (kb <= kb_last) block(kb, 0);
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

// The tiles come sorted by falling number of key blocks; with `pair`, workgroup x takes tile x and then tile n - 1 - x,
// so that every workgroup has about the same work (a causal prompt's last tile reads many times more keys than its first).
__global__ void __launch_bounds__(PF_THREADS)
LEV_NAME(attn_prefill_hd)(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long o_stride,
                          const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages,
                          const int* __restrict__ positions, const int* __restrict__ token_seq,
                          const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ tiles, int n_tiles, int pair,
                          int H, int KVH, int ps_shift, float scale, int window) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[4][NCHUNK][16][8];  // [score tile 2u+h][chunk][row][8]
  __shared__ __attribute__((aligned(16))) bf16_t Vs[HD][VS_STRIDE];
  const int first = blockIdx.x, second = n_tiles - 1 - blockIdx.x;
  prefill_tile(q, q_stride, out, o_stride, k_pages, v_pages, positions, token_seq, block_tables, bt_stride, tiles[2 * first],
               tiles[2 * first + 1], blockIdx.y, H, KVH, ps_shift, scale, window, Ks, Vs);
  if (pair && second > first)
    prefill_tile(q, q_stride, out, o_stride, k_pages, v_pages, positions, token_seq, block_tables, bt_stride, tiles[2 * second],
                 tiles[2 * second + 1], blockIdx.y, H, KVH, ps_shift, scale, window, Ks, Vs);
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
__global__ void __launch_bounds__(64 * DECODE_WG_WAVES)
LEV_NAME(attn_decode_hd)(const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long o_stride,
                         bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, const int* __restrict__ positions,
                         const int* __restrict__ token_seq, const int* __restrict__ block_tables, int bt_stride,
                         const int* __restrict__ decode_tokens, const bf16_t* __restrict__ k_new,
                         const bf16_t* __restrict__ v_new, long kv_stride, const int* __restrict__ dest,
                         float* __restrict__ ws_m, float* __restrict__ ws_l, float* __restrict__ ws_o,
                         int H, int KVH, int ps_shift, int splits, float scale, int window, int wg_merge) {
  const int PS = 1 << ps_shift, ps_mask = PS - 1;
  const float scale_log2 = scale * 1.4426950408889634f;
  const int lane = threadIdx.x & 63;
  const int fr = lane & 15, g = lane >> 4;
  const int idx = blockIdx.x, kvh = blockIdx.y, z = wg_merge ? (int)(threadIdx.x >> 6) : (int)blockIdx.z;
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
    uint32_t v_mask[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kp = key0 + 32 * u + 8 * g;
      const int page = vpg[u];
      v_mask[u] = (kp <= pos && kp + 7 >= lo && page >= 0) ? 0xffffffffu : 0u;
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
        u32x4 v = vf[dt][u] & u32x4{v_mask[u], v_mask[u], v_mask[u], v_mask[u]};
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
    softmax_block(st, scale_log2, q_pos, lo, key0, g, key0 + 63 > pos || key0 < lo, m, l, o, pf);
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
                                               int KVH, int PS, int splits, float scale, int window, hipStream_t stream) {
  int ps_shift = 0;
  while ((1 << ps_shift) < PS) ++ps_shift;
  if ((1 << ps_shift) != PS) return lev_fail("attention (matrix cores): page_size=%d must be a power of two", PS);
  if (n_prefill_tiles > 0) {
    // pairing halves the number of workgroups: only when every CU (256 of them) still gets one
    const int pair = (long)n_prefill_tiles * H >= 512;
    dim3 grid(pair ? (n_prefill_tiles + 1) / 2 : n_prefill_tiles, H);
    LEV_NAME(attn_prefill_hd)<<<grid, PF_THREADS, 0, stream>>>((const bf16_t*)q, q_stride, (bf16_t*)out, o_stride,
                                                        (const bf16_t*)k_pages, (const bf16_t*)v_pages, positions, token_seq,
                                                        block_tables, bt_stride, prefill_tiles, n_prefill_tiles, pair, H,
                                                        KVH, ps_shift, scale, window);
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
        splits, scale, window, wg_merge);
    if (int rc = lev_check_launch("attention decode")) return rc;
    if (splits > 1 && !wg_merge) {
      dim3 cgrid(n_decode, H);
      LEV_NAME(attn_combine_hd)<<<cgrid, 64, 0, stream>>>((bf16_t*)out, o_stride, decode_tokens, ws_m, ws_l, ws_o, H, splits);
      if (int rc = lev_check_launch("attention combine")) return rc;
    }
  }
  return 0;
}
