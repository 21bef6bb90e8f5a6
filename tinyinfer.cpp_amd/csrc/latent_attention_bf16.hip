// Latent attention in bfloat16 on the matrix cores of gfx950.
//
// A token's page row holds [c (R) | kr (r)], and the page holds the latents a second time transposed, [R][P], behind its P
// rows: the first product reduces over the R + r entries of a row, the second over the keys, and each reads its operand
// along the dimension it reduces over, straight from memory.  Every head attends over the same rows with its absorbed
// query qa = [W_uk^T q_plain | q_rot]; the weighted latent o goes through W_uv afterwards:
//   latent_absorb_mfma   qa^T (R x 16 tokens)   = W_uk_h^T (R x d) . q_plain^T      a wavefront per (16 tokens, head, 16 entries)
//   S^T (16 keys x 16 columns)                   = [c | kr] (16 x DK) . qa^T
//   O^T (R x 16 columns)                        += c^T (R x 32 keys) . P^T
//   latent_expand_mfma   out^T (dv x 16 tokens)  = W_uv_h (dv x R) . o^T
// all with v_mfma_f32_16x16x32_bf16.  The transposed score tile leaves each lane with four keys of one column, the layout
// the second product wants for P^T.  Scores, the running softmax and the sink (exp(sink_h) in the denominator only, added
// once when a column is finished) are 32-bit.
//
// What the 16 columns are: for a tile of a prompt's portion, 16 consecutive tokens of one head (a workgroup's four
// wavefronts take four such runs); for single rows (decoded tokens), 16 heads of one token, the four wavefronts taking the
// pairs of key blocks in turns and merging through LDS, and several workgroups sharing a long context with a merge kernel
// behind them.  A column at position p sees the keys max(0, p - window + 1) .. p (window 0: all).
//
// Sizes: the kernels are compiled for (k-steps of 32 over R + r, blocks of 16 over R) = (3, 4), (6, 8), (10, 16), (18, 32);
// a model takes the smallest that holds it, steps and blocks beyond its sizes are skipped.  R a multiple of 16, R + r and
// the unrotated query size multiples of 8, the value size a multiple of 16, pages of a multiple of 16 rows.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define LA_LOG2E 1.4426950408889634f

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) const u32x4 lds_u32x4;      // reads and writes that are known to go to LDS
typedef __attribute__((address_space(3))) u32x4 lds_w_u32x4;
typedef __attribute__((address_space(3))) u32x2 lds_w_u32x2;

union LFrag8 {
  uint4 u;
  u32x4 n;
  bf16x8 v;
};

struct LatPages {
  const bf16_t* pool;   // [pages][rows: [P][DK] | transposed latents: [R][P]]
  const int* table;     // block-table row of the request
  int P, DK, R;
  size_t page_elems;
};

template <int NRT>
struct LatState {
  float m, l;           // maximum (units of log 2) of the column; this lane's share of the sum of weights
  floatx4 o[NRT];       // O^T: rows (latent entries) 16 d + 4 (lane / 16) + i, column lane % 16
  __device__ __forceinline__ void clear() {
    m = -INFINITY;
    l = 0.f;
#pragma unroll
    for (int d = 0; d < NRT; ++d) o[d] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
};

// A pair of blocks in LDS, fetched once by a workgroup for its four wavefronts: the 32 key rows, padded by 16 bytes so that
// the fragments' reads spread over the banks, then the latents transposed: a row per entry that holds, quarter by quarter,
// four keys of the first block and the same four of the second: a lane's fragment in one read.
template <int NKS, int NRT>
struct LatStage {
  static constexpr int KROW = NKS * 32 + 8;
  static constexpr int VROW = 32 + 8;
  static constexpr int K_ELEMS = 32 * KROW;
  static constexpr int ELEMS = K_ELEMS + NRT * 16 * VROW;
  static constexpr int K_PIECES = 32 * NKS * 4;            // pieces of 16 bytes: 32 rows of NKS 4
  static constexpr int V_PIECES = NRT * 16 * 4;            // an entry's 8 keys of either half of either block
  static constexpr int NK = (K_PIECES + 255) / 256, NV = (V_PIECES + 255) / 256;
};

// One pair of blocks of 16 keys, [keyA, keyA + 16) and [keyA + 16, keyA + 32), for this wavefront's 16 columns.  `stage`:
// the pair as a workgroup left it in LDS (null: every wavefront reads its fragments from memory).
//   qf        qa^T fragments: column lane % 16, entries 32 s + 8 (lane / 16) .. + 7
//   lo, hi    the keys this lane's column sees: lo <= key <= hi (lo > hi: none)
//   lo_max, hi_min   the largest lo and the smallest hi of the wavefront's live columns
//   kv_last   last position of the request that has been written (rows after it hold anything, NaN included)
//   safe_key  a key whose page exists: loads of blocks that do not count go there, so that they never leave the pool
template <int NKS, int NRT, bool FROM_LDS>
__device__ __forceinline__ void latent_pair(const LatPages& kv, const LFrag8* qf, int keyA, int lo, int hi, int lo_max, int hi_min,
                                            int kv_last, int safe_key, float scale2, LatState<NRT>& st, const bf16_t* stage = nullptr) {
  const int lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int keyB = keyA + 16;
  int pageA = keyA <= kv_last ? kv.table[keyA / kv.P] : -1;
  int pageB = keyB <= kv_last ? kv.table[keyB / kv.P] : -1;
  const bool validA = pageA >= 0, validB = pageB >= 0;
  int rowA = keyA % kv.P, rowB = keyB % kv.P;
  if (!validA) {
    pageA = kv.table[safe_key / kv.P];
    rowA = (safe_key % kv.P) & ~15;
  }
  if (!validB) {
    pageB = kv.table[safe_key / kv.P];
    rowB = (safe_key % kv.P) & ~15;
  }
  const bool plain = validA && validB && keyA >= lo_max && keyB + 15 <= hi_min;
  // Every load is issued whatever the sizes (a step or block beyond them reads the last one that exists and counts as zero),
  // so that nothing stands between the loads and they are all in flight together.
  const bf16_t* ka = kv.pool + (size_t)pageA * kv.page_elems + (size_t)(rowA + r16) * kv.DK;
  const bf16_t* kb = kv.pool + (size_t)pageB * kv.page_elems + (size_t)(rowB + r16) * kv.DK;
  // the transposed latents: row (entry) 16 d + lane % 16, keys 4 (lane / 16) .. + 3 of either block
  const size_t t_base = (size_t)kv.P * kv.DK;
  const bf16_t* va = kv.pool + (size_t)pageA * kv.page_elems + t_base + rowA + quad * 4;
  const bf16_t* vb = kv.pool + (size_t)pageB * kv.page_elems + t_base + rowB + quad * 4;
  floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
  uint2 ta[NRT], tb[NRT];
  if (FROM_LDS) {      // LDS answers fast: a fragment is read where it is used
    using S = LatStage<NKS, NRT>;
#pragma unroll
    for (int s = 0; s < NKS; ++s) {
      LFrag8 a, b;
      a.n = *(lds_u32x4*)(size_t)(stage + r16 * S::KROW + s * 32 + quad * 8);
      b.n = *(lds_u32x4*)(size_t)(stage + (16 + r16) * S::KROW + s * 32 + quad * 8);
      if (!(s * 32 + quad * 8 < kv.DK)) a.u = b.u = make_uint4(0u, 0u, 0u, 0u);
      sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[s].v, sa, 0, 0, 0);
      sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.v, qf[s].v, sb, 0, 0, 0);
    }
  } else {
    LFrag8 fa[NKS], fb[NKS];
#pragma unroll
    for (int s = 0; s < NKS; ++s) {
      const int at = min(s * 32 + quad * 8, kv.DK - 8);
      fa[s].u = *reinterpret_cast<const uint4*>(ka + at);
      fb[s].u = *reinterpret_cast<const uint4*>(kb + at);
    }
#pragma unroll
    for (int s = 0; s < NKS; ++s) {
      if (!(s * 32 + quad * 8 < kv.DK)) fa[s].u = fb[s].u = make_uint4(0u, 0u, 0u, 0u);
      sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[s].v, qf[s].v, sa, 0, 0, 0);
      sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[s].v, qf[s].v, sb, 0, 0, 0);
    }
#pragma unroll
    for (int d = 0; d < NRT; ++d) {
      const int c = min(d * 16 + r16, kv.R - 1);
      ta[d] = *reinterpret_cast<const uint2*>(va + (size_t)c * kv.P);
      tb[d] = *reinterpret_cast<const uint2*>(vb + (size_t)c * kv.P);
    }
  }
  float sv[8];
  unsigned keepA[2] = {0xFFFFFFFFu, 0xFFFFFFFFu}, keepB[2] = {0xFFFFFFFFu, 0xFFFFFFFFu};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int ja = keyA + quad * 4 + i, jb = keyB + quad * 4 + i;
    const bool see_a = plain || (validA & (ja >= lo) & (ja <= hi));
    const bool see_b = plain || (validB & (jb >= lo) & (jb <= hi));
    sv[i] = see_a ? sa[i] * scale2 : -INFINITY;
    sv[4 + i] = see_b ? sb[i] * scale2 : -INFINITY;
    if (!plain) {
      // 0 * NaN is NaN: latents of rows that were never written (or of a stand-in page) become zero
      const unsigned half = (i & 1) ? 0x0000FFFFu : 0xFFFF0000u;
      if (!validA | (ja > kv_last)) keepA[i >> 1] &= half;
      if (!validB | (jb > kv_last)) keepB[i >> 1] &= half;
    }
  }
  float bm = sv[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) bm = fmaxf(bm, sv[i]);
  bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
  bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
  const float m_new = fmaxf(st.m, bm);
  const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
  float pv[8], ps = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    pv[i] = __builtin_amdgcn_exp2f(sv[i] - m_safe);
    ps += pv[i];
  }
  LFrag8 pf;
  pf.u = make_uint4(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]), pack_bf16x2(pv[4], pv[5]), pack_bf16x2(pv[6], pv[7]));
  if (__builtin_amdgcn_ballot_w64(m_new != st.m) != 0) {
    const float alpha = __builtin_amdgcn_exp2f(st.m - m_safe);      // m = -inf: 0, and l and o are 0 anyway
    st.l *= alpha;
#pragma unroll
    for (int d = 0; d < NRT; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i) st.o[d][i] *= alpha;
    st.m = m_new;
  }
  st.l += ps;
#pragma unroll
  for (int d = 0; d < NRT; ++d) {
    const bool in = d * 16 + r16 < kv.R;      // a row beyond the latent: the output's rows there are never stored
    if (FROM_LDS) {
      const u32x4 t = *(lds_u32x4*)(size_t)(stage + LatStage<NKS, NRT>::K_ELEMS + (d * 16 + r16) * LatStage<NKS, NRT>::VROW + quad * 8);
      ta[d] = make_uint2(t[0], t[1]);
      tb[d] = make_uint2(t[2], t[3]);
    }
    LFrag8 v;
    v.u = make_uint4(ta[d].x & keepA[0], ta[d].y & keepA[1], tb[d].x & keepB[0], tb[d].y & keepB[1]);
    if (!in) v.u = make_uint4(0u, 0u, 0u, 0u);
    st.o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v.v, pf.v, st.o[d], 0, 0, 0);
  }
}

// the absorbed query of this lane's column: qa row [DK], entries 32 s + 8 (lane / 16) .. + 7
template <int NKS>
__device__ __forceinline__ void load_query(const bf16_t* qrow, int DK, LFrag8* qf) {
  const int quad = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int s = 0; s < NKS; ++s) {
    qf[s].u = *reinterpret_cast<const uint4*>(qrow + min(s * 32 + quad * 8, DK - 8));
    if (!(s * 32 + quad * 8 < DK)) qf[s].u = make_uint4(0u, 0u, 0u, 0u);
  }
}

// the column's weighted latent divided by its sum of weights, the sink in the sum: o bf16 [R] of the column
template <int NRT>
__device__ __forceinline__ void finish_column(LatState<NRT>& st, const float* sink, int h, int R, bf16_t* dst, bool live) {
  const int quad = (threadIdx.x & 63) >> 4;
  float l = st.l;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  const float s2 = sink ? sink[h] * LA_LOG2E : -INFINITY;
  const float mm = fmaxf(st.m, s2);
  const float m_safe = (mm == -INFINITY) ? 0.f : mm;
  const float a = __builtin_amdgcn_exp2f(st.m - m_safe);
  const float lt = l * a + (sink ? __builtin_amdgcn_exp2f(s2 - m_safe) : 0.f);
  const float f = lt > 0.f ? a / lt : 0.f;
  if (!live) return;
#pragma unroll
  for (int d = 0; d < NRT; ++d)
    if (d * 16 < R)
      *reinterpret_cast<uint2*>(dst + d * 16 + quad * 4) =
          make_uint2(pack_bf16x2(st.o[d][0] * f, st.o[d][1] * f), pack_bf16x2(st.o[d][2] * f, st.o[d][3] * f));
}

// ------------------------------------------------------------------------------------------ tiles of a portion
// tiles int32 [n][3] = (entry, first row, rows <= 64); entries int32 [.][4] = (row0, tokens, start, -).  qa [M][H][DK],
// o [M][H][R].  Grid (heads, tiles), four wavefronts of 16 rows each.
template <int NKS, int NRT>
__global__ void __launch_bounds__(256)
latent_tiles_kernel(const bf16_t* __restrict__ qa, const bf16_t* __restrict__ pool, const int* __restrict__ table, int table_stride,
                    const int* __restrict__ tiles, const int* __restrict__ entries, const float* __restrict__ sink,
                    bf16_t* __restrict__ o, int H, int R, int DK, int P, size_t page_elems, float scale2, int window) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15;
  const int e = tiles[3 * blockIdx.y], row0 = tiles[3 * blockIdx.y + 1] + 16 * wave;
  const int n_rows = tiles[3 * blockIdx.y + 2] - 16 * wave;
  if (n_rows <= 0) return;
  const int h = blockIdx.x;
  const int e_row0 = entries[4 * e], e_n = entries[4 * e + 1], e_start = entries[4 * e + 2];
  const int kv_last = e_start + e_n - 1;
  const bool live = r16 < n_rows;
  const int row = row0 + (live ? r16 : 0);
  const int p = e_start + (row - e_row0);
  const int lo_p = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int lo = live ? lo_p : 1, hi = live ? p : 0;
  int lo_min = live ? lo : 0x7fffffff, lo_max = live ? lo : 0, hi_min = live ? hi : 0x7fffffff, hi_max = hi;
#pragma unroll
  for (int x = 1; x < 16; x <<= 1) {
    lo_min = min(lo_min, __shfl_xor(lo_min, x, 64));
    lo_max = max(lo_max, __shfl_xor(lo_max, x, 64));
    hi_min = min(hi_min, __shfl_xor(hi_min, x, 64));
    hi_max = max(hi_max, __shfl_xor(hi_max, x, 64));
  }
  LatPages kv{pool, table + (size_t)e * table_stride, P, DK, R, page_elems};
  LFrag8 qf[NKS];
  load_query<NKS>(qa + ((size_t)row * H + h) * DK, DK, qf);
  LatState<NRT> st;
  st.clear();
  for (int pr = lo_min / 32; pr <= hi_max / 32; ++pr)
    latent_pair<NKS, NRT, false>(kv, qf, pr * 32, lo, hi, lo_max, hi_min, kv_last, hi_max, scale2, st);
  finish_column<NRT>(st, sink, h, R, o + ((size_t)row * H + h) * R, live);
}

// ------------------------------------------------------------------------------------------ tiles, the pairs through LDS
// The same tiles with the four wavefronts sharing what they read: a pair of blocks is fetched once by the workgroup into one
// of two LDS stages (through registers: thread t the 16-byte pieces t, t + 256, ...) while the pair before it is multiplied
// from the other; one barrier a pair.
template <int NKS, int NRT>
__device__ __forceinline__ void fetch_pair(const LatPages& kv, int keyA, int kv_last, int safe_key, u32x4* __restrict__ fk, u32x4* __restrict__ fv) {
  using S = LatStage<NKS, NRT>;
  const int keyB = keyA + 16;
  int pageA = keyA <= kv_last ? kv.table[keyA / kv.P] : -1;
  int pageB = keyB <= kv_last ? kv.table[keyB / kv.P] : -1;
  int rowA = keyA % kv.P, rowB = keyB % kv.P;
  if (pageA < 0) {
    pageA = kv.table[safe_key / kv.P];
    rowA = (safe_key % kv.P) & ~15;
  }
  if (pageB < 0) {
    pageB = kv.table[safe_key / kv.P];
    rowB = (safe_key % kv.P) & ~15;
  }
  const bf16_t* pa = kv.pool + (size_t)pageA * kv.page_elems;
  const bf16_t* pb = kv.pool + (size_t)pageB * kv.page_elems;
#pragma unroll
  for (int j = 0; j < S::NK; ++j) {
    const int idx = min((int)threadIdx.x + 256 * j, S::K_PIECES - 1);
    const int row = idx / (NKS * 4), pc = idx % (NKS * 4);
    const bf16_t* src = (row < 16 ? pa + (size_t)(rowA + row) * kv.DK : pb + (size_t)(rowB + row - 16) * kv.DK) + min(pc * 8, kv.DK - 8);
    fk[j] = *reinterpret_cast<const u32x4*>(src);
  }
  const size_t t_base = (size_t)kv.P * kv.DK;
#pragma unroll
  for (int j = 0; j < S::NV; ++j) {
    const int idx = min((int)threadIdx.x + 256 * j, S::V_PIECES - 1);
    const int c = min(idx >> 2, kv.R - 1), blk = (idx >> 1) & 1, half = idx & 1;
    const bf16_t* src = (blk ? pb + rowB : pa + rowA) + t_base + (size_t)c * kv.P + half * 8;
    fv[j] = *reinterpret_cast<const u32x4*>(src);
  }
}

template <int NKS, int NRT>
__device__ __forceinline__ void stash_pair(bf16_t* stage, const u32x4* __restrict__ fk, const u32x4* __restrict__ fv) {
  using S = LatStage<NKS, NRT>;
#pragma unroll
  for (int j = 0; j < S::NK; ++j) {
    const int idx = threadIdx.x + 256 * j;
    if (idx < S::K_PIECES) *(lds_w_u32x4*)(size_t)(stage + (idx / (NKS * 4)) * S::KROW + (idx % (NKS * 4)) * 8) = fk[j];
  }
#pragma unroll
  for (int j = 0; j < S::NV; ++j) {
    const int idx = threadIdx.x + 256 * j;
    if (idx < S::V_PIECES) {
      const int c = idx >> 2, blk = (idx >> 1) & 1, half = idx & 1;
      bf16_t* dst = stage + S::K_ELEMS + c * S::VROW + blk * 4;      // keys 8 half .. + 7: the quarters 2 half and 2 half + 1
      *(lds_w_u32x2*)(size_t)(dst + (2 * half) * 8) = u32x2{fv[j][0], fv[j][1]};
      *(lds_w_u32x2*)(size_t)(dst + (2 * half + 1) * 8) = u32x2{fv[j][2], fv[j][3]};
    }
  }
}

template <int NKS, int NRT>
__global__ void __launch_bounds__(256)
latent_tiles_lds_kernel(const bf16_t* __restrict__ qa, const bf16_t* __restrict__ pool, const int* __restrict__ table, int table_stride,
                        const int* __restrict__ tiles, const int* __restrict__ entries, const float* __restrict__ sink,
                        bf16_t* __restrict__ o, int H, int R, int DK, int P, size_t page_elems, float scale2, int window) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  bf16_t* stages = reinterpret_cast<bf16_t*>(lds_raw);
  using S = LatStage<NKS, NRT>;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15;
  const int e = tiles[3 * blockIdx.y], tile_row0 = tiles[3 * blockIdx.y + 1], tile_n = tiles[3 * blockIdx.y + 2];
  const int row0 = tile_row0 + 16 * wave, n_rows = tile_n - 16 * wave;      // a wavefront without rows still fetches and waits
  const int h = blockIdx.x;
  const int e_row0 = entries[4 * e], e_n = entries[4 * e + 1], e_start = entries[4 * e + 2];
  const int kv_last = e_start + e_n - 1;
  const bool live = r16 < n_rows;
  const int row = live ? row0 + r16 : tile_row0;
  const int p = e_start + (row - e_row0);
  const int lo_p = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int lo = live ? lo_p : 1, hi = live ? p : 0;
  int lo_min = live ? lo : 0x7fffffff, lo_max = live ? lo : 0, hi_min = live ? hi : 0x7fffffff, hi_max = live ? hi : -1;
#pragma unroll
  for (int x = 1; x < 16; x <<= 1) {
    lo_min = min(lo_min, __shfl_xor(lo_min, x, 64));
    lo_max = max(lo_max, __shfl_xor(lo_max, x, 64));
    hi_min = min(hi_min, __shfl_xor(hi_min, x, 64));
    hi_max = max(hi_max, __shfl_xor(hi_max, x, 64));
  }
  // the workgroup's keys: from the first one its first row sees to its last row's own
  const int p_first = e_start + (tile_row0 - e_row0), p_last = p_first + tile_n - 1;
  const int first = ((window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0) / 32, last = p_last / 32;
  LatPages kv{pool, table + (size_t)e * table_stride, P, DK, R, page_elems};
  LFrag8 qf[NKS];
  load_query<NKS>(qa + ((size_t)row * H + h) * DK, DK, qf);
  LatState<NRT> st;
  st.clear();
  u32x4 fk[S::NK], fv[S::NV];
  fetch_pair<NKS, NRT>(kv, first * 32, kv_last, p_last, fk, fv);
  stash_pair<NKS, NRT>(stages, fk, fv);
  __syncthreads();
  for (int pr = first; pr <= last; ++pr) {
    const bf16_t* cur = stages + ((pr - first) & 1) * S::ELEMS;
    bf16_t* nxt = stages + ((pr - first + 1) & 1) * S::ELEMS;
    // (behind the last pair the same pair is fetched and stashed once more, into the stage nobody reads any longer)
    fetch_pair<NKS, NRT>(kv, min(pr + 1, last) * 32, kv_last, p_last, fk, fv);
    if (pr * 32 <= hi_max && pr * 32 + 31 >= lo_min)
      latent_pair<NKS, NRT, true>(kv, qf, pr * 32, lo, hi, lo_max, hi_min, kv_last, p_last, scale2, st, cur);
    stash_pair<NKS, NRT>(nxt, fk, fv);
    __syncthreads();
  }
  finish_column<NRT>(st, sink, h, R, o + ((size_t)row * H + h) * R, live);
}

// ------------------------------------------------------------------------------------------ single rows
// rows int32 [n] (null: row r is r); the 16 columns are the heads 16 blockIdx.y .. + 15 of the row's token.  Workgroup z of
// gridDim.z, wavefront v take the pairs of blocks 4 z + v, 4 z + v + 4 gridDim.z, ...; the wavefronts merge through LDS in
// the order 1, 2, 3.  One workgroup a row finishes the columns; several leave their shares in `part`.
template <int NRT>
__device__ __forceinline__ void merge_share(LatState<NRT>& st, const float* src, int lane) {
  const float m2 = src[NRT * 4 * 64 + lane], l2 = src[(NRT * 4 + 1) * 64 + lane];
  const float mm = fmaxf(st.m, m2);
  const float m_safe = (mm == -INFINITY) ? 0.f : mm;
  const float a = __builtin_amdgcn_exp2f(st.m - m_safe), b = __builtin_amdgcn_exp2f(m2 - m_safe);
  st.l = st.l * a + l2 * b;
#pragma unroll
  for (int d = 0; d < NRT; ++d)
#pragma unroll
    for (int i = 0; i < 4; ++i) st.o[d][i] = st.o[d][i] * a + src[(d * 4 + i) * 64 + lane] * b;
  st.m = mm;
}

template <int NRT>
__device__ __forceinline__ void store_share(const LatState<NRT>& st, float* dst, int lane) {
#pragma unroll
  for (int d = 0; d < NRT; ++d)
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[(d * 4 + i) * 64 + lane] = st.o[d][i];
  dst[NRT * 4 * 64 + lane] = st.m;
  dst[(NRT * 4 + 1) * 64 + lane] = st.l;
}

template <int NKS, int NRT>
__global__ void __launch_bounds__(256)
latent_rows_mfma_kernel(const bf16_t* __restrict__ qa, const bf16_t* __restrict__ pool, const int* __restrict__ table, int table_stride,
                        const int* __restrict__ pos, const int* __restrict__ slot, const int* __restrict__ rows,
                        const float* __restrict__ sink, bf16_t* __restrict__ o, int H, int R, int DK, int P, size_t page_elems,
                        float scale2, int window, float* __restrict__ part, int n_splits) {
  extern __shared__ float lds[];     // [NRT 4 + 2][64]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15;
  const int m = rows ? rows[blockIdx.x] : blockIdx.x;
  const int p = pos[m];
  const bool live = (int)blockIdx.y * 16 + r16 < H;
  const int h = live ? blockIdx.y * 16 + r16 : 0;
  const int lo_all = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int lo = live ? lo_all : 1, hi = live ? p : 0;
  LatPages kv{pool, table + (size_t)slot[m] * table_stride, P, DK, R, page_elems};
  LFrag8 qf[NKS];
  load_query<NKS>(qa + ((size_t)m * H + h) * DK, DK, qf);
  LatState<NRT> st;
  st.clear();
  for (int pr = lo_all / 32 + 4 * blockIdx.z + wave; pr <= p / 32; pr += 4 * n_splits)
    latent_pair<NKS, NRT, false>(kv, qf, pr * 32, lo, hi, lo_all, p, p, p, scale2, st);
  for (int w = 1; w < 4; ++w) {
    if (wave == w) store_share<NRT>(st, lds, lane);
    __syncthreads();
    if (wave == 0) merge_share<NRT>(st, lds, lane);
    __syncthreads();
  }
  if (wave > 0) return;
  if (n_splits == 1) {
    finish_column<NRT>(st, sink, h, R, o + ((size_t)m * H + h) * R, live);
    return;
  }
  store_share<NRT>(st, part + (((size_t)blockIdx.x * gridDim.y + blockIdx.y) * n_splits + blockIdx.z) * (NRT * 4 + 2) * 64, lane);
}

// The shares of the workgroups that split a row's keys, added up.  Grid (rows, groups of 16 heads, NRT): a wavefront owns one
// entry of every column's four (its lanes as the shares lie in memory), works out every share's weight itself (the sink joins
// the maximum and the sum there) and adds its entries up, shares ascending.
template <int NRT>
__global__ void __launch_bounds__(256)
latent_rows_merge_kernel(const float* __restrict__ part, const int* __restrict__ rows, const float* __restrict__ sink,
                         bf16_t* __restrict__ o, int H, int R, int n_splits) {
  constexpr int PER = (NRT * 4 + 2) * 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int m = rows ? rows[blockIdx.x] : blockIdx.x;
  const bool live = (int)blockIdx.y * 16 + r16 < H;
  const int h = live ? blockIdx.y * 16 + r16 : 0;
  const int idx = blockIdx.z * 4 + wave;
  const float* base = part + ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * n_splits * PER + lane;
  const float s2 = sink ? sink[h] * LA_LOG2E : -INFINITY;
  float mm = s2;
#pragma unroll 8
  for (int s = 0; s < n_splits; ++s) mm = fmaxf(mm, base[(size_t)s * PER + NRT * 4 * 64]);
  const float m_safe = (mm == -INFINITY) ? 0.f : mm;
  float l = 0.f, acc = 0.f;
#pragma unroll 8
  for (int s = 0; s < n_splits; ++s) {
    const float w = __builtin_amdgcn_exp2f(base[(size_t)s * PER + NRT * 4 * 64] - m_safe);
    l = fmaf(base[(size_t)s * PER + (NRT * 4 + 1) * 64], w, l);
    acc = fmaf(base[(size_t)s * PER + idx * 64], w, acc);
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  const float lt = l + (sink ? __builtin_amdgcn_exp2f(s2 - m_safe) : 0.f);
  const int c = (idx >> 2) * 16 + quad * 4 + (idx & 3);
  if (live && c < R) o[((size_t)m * H + h) * R + c] = f2bf(lt > 0.f ? acc / lt : 0.f);
}

// ------------------------------------------------------------------------------------------ the absorbed query
// qa [M][H][DK] bf16: entries c < R: sum_k q[m, h, k] W_uk[h d + k, c], from w_uk_t [H][R][d] (a head's matrix transposed);
// entries R + j: q_rot[m, h, j].  proj f32 [M, ld] holds the heads' queries [d + r] from column 0.  Grid (tokens / 16, heads,
// R / 256): a wavefront takes four blocks of 16 latent entries.  A step of the sum beyond d reads the last one and counts as zero.
__global__ void __launch_bounds__(256)
latent_absorb_mfma_kernel(const float* __restrict__ proj, int ldp, const bf16_t* __restrict__ w_uk_t, bf16_t* __restrict__ qa, int M,
                          int H, int d, int r, int R) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int h = blockIdx.y, DK = R + r;
  const int tok = blockIdx.x * 16 + r16;
  const bool live = tok < M;
  const float* q = proj + (size_t)(live ? tok : M - 1) * ldp + (size_t)h * (d + r);
  // a wavefront takes four blocks of 16 latent entries: a step's query fragment is fetched once for the four
  const int ct0 = (blockIdx.z * 4 + wave) * 4;
  if (ct0 * 16 < R) {
    const bf16_t* w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = w_uk_t + ((size_t)h * R + min((ct0 + j) * 16 + r16, R - 1)) * d;
    floatx4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
    for (int k0 = 0; k0 < d; k0 += 32) {
      const int at = min(k0 + quad * 8, d - 8);
      const bool in = k0 + quad * 8 < d;
      const float4 x = *reinterpret_cast<const float4*>(q + at), y = *reinterpret_cast<const float4*>(q + at + 4);
      LFrag8 b;
      b.u = make_uint4(pack_bf16x2(x.x, x.y), pack_bf16x2(x.z, x.w), pack_bf16x2(y.x, y.y), pack_bf16x2(y.z, y.w));
      if (!in) b.u = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        LFrag8 a;
        a.u = *reinterpret_cast<const uint4*>(w[j] + at);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[j], 0, 0, 0);
      }
    }
    if (live)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if ((ct0 + j) * 16 < R)
          *reinterpret_cast<uint2*>(qa + ((size_t)tok * H + h) * DK + (ct0 + j) * 16 + quad * 4) =
              make_uint2(pack_bf16x2(acc[j][0], acc[j][1]), pack_bf16x2(acc[j][2], acc[j][3]));
  }
  if (blockIdx.z == 0) {
    const int n = min(16, M - (int)blockIdx.x * 16);
    for (int e = threadIdx.x; e < n * r; e += 256) {
      const int t = blockIdx.x * 16 + e / r, j = e % r;
      qa[((size_t)t * H + h) * DK + R + j] = f2bf(proj[(size_t)t * ldp + (size_t)h * (d + r) + d + j]);
    }
  }
}

// ------------------------------------------------------------------------------------------ a head's weighted latent to its output
// out [M][H dv] bf16: out[m, h dv + j] = sum_c o[m, h, c] W_uv[h dv + j, c].  Grid (tokens / 16, heads, dv / 128): a wavefront
// takes two blocks of 16 outputs.
__global__ void __launch_bounds__(256)
latent_expand_mfma_kernel(const bf16_t* __restrict__ o, const bf16_t* __restrict__ w_uv, bf16_t* __restrict__ out, int M, int H, int R,
                          int dv) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, quad = lane >> 4;
  const int h = blockIdx.y;
  const int tok = blockIdx.x * 16 + r16;
  const bool live = tok < M;
  // a wavefront takes two blocks of 16 outputs: a step's fragment of the weighted latent is fetched once for both
  const int jt0 = (blockIdx.z * 4 + wave) * 2;
  if (jt0 * 16 >= dv) return;
  const bf16_t* orow = o + ((size_t)(live ? tok : M - 1) * H + h) * R;
  const bf16_t* w[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) w[j] = w_uv + ((size_t)h * dv + min((jt0 + j) * 16 + r16, dv - 1)) * R;
  floatx4 acc[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll 4
  for (int c0 = 0; c0 < R; c0 += 32) {
    const int at = min(c0 + quad * 8, R - 8);
    LFrag8 b;
    b.u = *reinterpret_cast<const uint4*>(orow + at);
    if (!(c0 + quad * 8 < R)) b.u = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      LFrag8 a;
      a.u = *reinterpret_cast<const uint4*>(w[j] + at);
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[j], 0, 0, 0);
    }
  }
  if (live)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      if ((jt0 + j) * 16 < dv)
        *reinterpret_cast<uint2*>(out + (size_t)tok * H * dv + (size_t)h * dv + (jt0 + j) * 16 + quad * 4) =
            make_uint2(pack_bf16x2(acc[j][0], acc[j][1]), pack_bf16x2(acc[j][2], acc[j][3]));
}

// ------------------------------------------------------------------------------------------ host
extern "C" int ti_latent_bf16_served(int H, int d, int r, int R, int dv, int page_size) {
  return H > 0 && d > 0 && d % 8 == 0 && (d + r) % 4 == 0 && r >= 0 && R > 0 && R % 16 == 0 && R <= 512 && (R + r) % 8 == 0 && R + r <= 576 && dv > 0 &&
         dv % 16 == 0 && page_size > 0 && page_size % 16 == 0;
}

#define LA_DISPATCH(CALL)                                         \
  do {                                                            \
    if (DK <= 96 && R <= 64) { CALL(3, 4); }                      \
    else if (DK <= 192 && R <= 128) { CALL(6, 8); }               \
    else if (DK <= 320 && R <= 256) { CALL(10, 16); }             \
    else { CALL(18, 32); }                                        \
  } while (0)

static int rows_block(int DK, int R) {
  if (DK <= 96 && R <= 64) return 4;
  if (DK <= 192 && R <= 128) return 8;
  if (DK <= 320 && R <= 256) return 16;
  return 32;
}

extern "C" int ti_latent_absorb_bf16(const float* proj, int ld, const void* w_uk_t, void* qa, int M, int H, int d, int r, int R,
                                     hipStream_t stream) {
  TI_REQUIRE(H > 0 && H <= 65535 && d > 0 && d % 8 == 0 && r >= 0 && R > 0 && R % 16 == 0 && ld >= H * (d + r) && ld % 4 == 0 &&
                 (d + r) % 4 == 0,
             "latent_absorb (bf16): bad sizes heads=%d dim=%d rot=%d rank=%d ld=%d", H, d, r, R, ld);
  if (M == 0) return 0;
  latent_absorb_mfma_kernel<<<dim3((M + 15) / 16, H, (R + 255) / 256), 256, 0, stream>>>(proj, ld, (const bf16_t*)w_uk_t, (bf16_t*)qa, M, H, d, r, R);
  TI_LAUNCH_CHECK();
  return 0;
}

extern "C" int ti_latent_expand_bf16(const void* o, const void* w_uv, void* out, int M, int H, int R, int dv, hipStream_t stream) {
  TI_REQUIRE(H > 0 && H <= 65535 && R > 0 && R % 8 == 0 && dv > 0 && dv % 16 == 0, "latent_expand (bf16): bad sizes heads=%d rank=%d vdim=%d", H, R, dv);
  if (M == 0) return 0;
  latent_expand_mfma_kernel<<<dim3((M + 15) / 16, H, (dv + 127) / 128), 256, 0, stream>>>((const bf16_t*)o, (const bf16_t*)w_uv, (bf16_t*)out, M, H, R, dv);
  TI_LAUNCH_CHECK();
  return 0;
}

// pool bf16 [pages][P rows of R + r | R rows of P]: page_elems elements a page
extern "C" int ti_latent_attention_tiles_bf16(const void* qa, const void* pool, long page_elems, const int* table, int table_stride,
                                              const int* tiles, const int* entries, const float* sink, void* o, int n_tiles, int H,
                                              int R, int r, int page_size, float scale, int window, int use_lds, hipStream_t stream) {
  const int DK = R + r;
  TI_REQUIRE(ti_latent_bf16_served(H, 8, 0, R, 16, page_size) && (R + r) % 8 == 0 && R + r <= 576 && H <= 65535 && table_stride > 0 && window >= 0 &&
                 page_elems >= (long)page_size * (DK + R),
             "latent_attention (tiles): heads=%d, a latent of %d + %d, pages of %d rows and %ld elements are not served", H, R, r,
             page_size, page_elems);
  if (n_tiles == 0) return 0;
  // heads along x: workgroups start in the order of the tiles' list, the ones that walk the most keys first, and the short
  // ones fill the compute units as the long ones end
  TI_REQUIRE(n_tiles <= 65535, "latent_attention (tiles): %d tiles in a step are not served", n_tiles);
  const dim3 grid(H, n_tiles);
  // keys and latents shared through LDS (use_lds 0: every wavefront fetches its own, for tests and measurements); the two
  // stages of the largest sizes need more than the 64 KB a kernel may use without asking
#define LA_TILES(K, V)                                                                                                              \
  do {                                                                                                                              \
    if (use_lds) {                                                                                                                  \
      const int bytes = 2 * LatStage<K, V>::ELEMS * 2;                                                                              \
      static bool asked = false;                                                                                                    \
      if (!asked && bytes > 64 * 1024) {                                                                                            \
        TI_REQUIRE(hipFuncSetAttribute((const void*)latent_tiles_lds_kernel<K, V>, hipFuncAttributeMaxDynamicSharedMemorySize,      \
                                       bytes) == hipSuccess, "latent_attention (tiles): %d bytes of LDS are refused", bytes);       \
        asked = true;                                                                                                               \
      }                                                                                                                             \
      latent_tiles_lds_kernel<K, V><<<grid, 256, bytes, stream>>>((const bf16_t*)qa, (const bf16_t*)pool, table, table_stride,      \
                                                                  tiles, entries, sink, (bf16_t*)o, H, R, DK, page_size,           \
                                                                  (size_t)page_elems, scale * LA_LOG2E, window);                    \
    } else {                                                                                                                        \
      latent_tiles_kernel<K, V><<<grid, 256, 0, stream>>>((const bf16_t*)qa, (const bf16_t*)pool, table, table_stride, tiles,       \
                                                          entries, sink, (bf16_t*)o, H, R, DK, page_size, (size_t)page_elems,       \
                                                          scale * LA_LOG2E, window);                                                \
    }                                                                                                                               \
  } while (0)
  LA_DISPATCH(LA_TILES);
#undef LA_TILES
  TI_LAUNCH_CHECK();
  return 0;
}

extern "C" int ti_latent_attention_rows_bf16(const void* qa, const void* pool, long page_elems, const int* table, int table_stride,
                                             const int* pos, const int* slot, const int* rows, const float* sink, void* o, int n_rows,
                                             int H, int R, int r, int page_size, float scale, int window, float* part, int n_splits,
                                             hipStream_t stream) {
  const int DK = R + r;
  TI_REQUIRE(ti_latent_bf16_served(H, 8, 0, R, 16, page_size) && (R + r) % 8 == 0 && R + r <= 576 && table_stride > 0 && window >= 0 && page_elems >= (long)page_size * (DK + R),
             "latent_attention (rows): heads=%d, a latent of %d + %d, pages of %d rows and %ld elements are not served", H, R, r, page_size,
             page_elems);
  TI_REQUIRE(n_splits >= 1 && n_splits <= 64 && (n_splits == 1 || part), "latent_attention (rows): %d splits need scratch", n_splits);
  if (n_rows == 0) return 0;
  const int groups = (H + 15) / 16;
  TI_REQUIRE(groups <= 65535, "latent_attention (rows): %d heads are not served", H);
  const dim3 grid(n_rows, groups, n_splits);
  const size_t lds = (size_t)(rows_block(DK, R) * 4 + 2) * 64 * 4;
#define LA_ROWS(K, V)                                                                                                              \
  latent_rows_mfma_kernel<K, V><<<grid, 256, lds, stream>>>((const bf16_t*)qa, (const bf16_t*)pool, table, table_stride, pos, slot, rows, \
                                                            sink, (bf16_t*)o, H, R, DK, page_size, (size_t)page_elems, scale * LA_LOG2E, \
                                                            window, part, n_splits)
  LA_DISPATCH(LA_ROWS);
#undef LA_ROWS
  TI_LAUNCH_CHECK();
  if (n_splits > 1) {
#define LA_MERGE(K, V) latent_rows_merge_kernel<V><<<dim3(n_rows, groups, V), 256, 0, stream>>>(part, rows, sink, (bf16_t*)o, H, R, n_splits)
    LA_DISPATCH(LA_MERGE);
#undef LA_MERGE
    TI_LAUNCH_CHECK();
  }
  return 0;
}

// floats of scratch for ti_latent_attention_rows_bf16 with n_splits > 1
extern "C" long ti_latent_attention_rows_scratch(int n_rows, int H, int R, int r, int n_splits) {
  return (long)n_rows * ((H + 15) / 16) * n_splits * (rows_block(R + r, R) * 4 + 2) * 64;
}
