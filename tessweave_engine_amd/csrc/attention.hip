// Attention over the paged cache, grouped-query, for float32 and bfloat16.
//
//   keys   [pages][kv_heads][page_size][head_dim]
//   values [pages][kv_heads][head_dim][page_size]   (transposed inside a page)
//   block_table[seq][b] = physical page of logical block b, or -1 if not held
//
// A query at absolute position t of a sequence with kv_len cached keys sees key
// p iff p <= t, p < kv_len and (window == 0 or p > t - window). Scores are
// q.k * scale; softmax statistics, probabilities and the output sum are float32.
// Masked scores are SELECTED to -inf and keys outside the sequence are loaded
// as zeros, so whatever an unowned or reused page holds (NaN included) never
// reaches a result.
//
// The unit of work is a wave with a tile of 16 query ROWS that share one kv
// head; a row is a (token, query head of the group) pair. Per 16 keys the wave
// computes S^T = K Q^T on the MFMA units (accumulator element j of lane
// (r, g) is the score of row r against key 4g + j), does the online-softmax
// update per row, and feeds the probabilities, still in accumulator layout, as
// the B operand of O^T += V^T P^T. Values are stored transposed in the page so
// that the A operand of that product is one aligned load of 4 consecutive keys.
//
//   attn_decode_kernel   rows = the group's heads of ONE token; the sequence's
//                        keys are split over workgroups (and over the 4 waves
//                        of each); partial results are merged in a fixed order.
//   attn_prefill_kernel  rows = (token, head) pairs of a prompt portion; each
//                        wave walks the keys its rows can see.
#include "tw_common.h"

template <typename T> __device__ __forceinline__ float tw_exp(float v);
template <> __device__ __forceinline__ float tw_exp<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ float tw_exp<bf16_t>(float v) { return __expf(v); }

template <typename T> struct KeyQuad;          // 4 consecutive keys of one d (A operand of the PV product)
template <> struct KeyQuad<float> { typedef f32x4 Type; };
template <> struct KeyQuad<bf16_t> { typedef bf16x4 Type; };

template <typename T, int DTMAX> struct AttnShape {
  static constexpr int EPF = Elem<T>::kPerFrag;
  static constexpr int NSMAX = (DTMAX * 16 / EPF + 3) / 4;    // MFMA steps over head_dim
};

struct AttnArgs {
  const void* q;          // [rows][ldq], head h of row n at q + n*ldq + h*head_dim
  long ldq;
  const void* keys;
  const void* values;
  const int* block_table;
  int table_stride;
  const int* q_start;     // [n_seqs + 1] first token row of each sequence
  const int* kv_len;      // [n_seqs] keys cached, this step's tokens included
  int seq0;               // first sequence this launch covers
  void* out;              // [rows][ldo]
  long ldo;
  float* part_o;          // decode partials [seq - seq0][q_heads][splits][head_dim]
  float* part_ml;         // [seq - seq0][q_heads][splits][2]  (max, sum)
  int q_heads, kv_heads, head_dim, page_size, window;
  float scale;
  float softcap;          // > 0: scores (after the scale) pass through softcap * tanh(score / softcap); the kernels
                          // that take every type and page size only
  int splits;
  int page_shift;         // log2(page_size) if it is a power of two, else -1
  int n_seqs, max_tiles;  // prefill (bfloat16 kernel): sequences of the launch, row tiles of the longest
  int tile_rows;          // rows of such a tile: 128, or 64 when there would be too few workgroups
  int kv_chunk, max_chunks;  // prefill (bfloat16 kernel): keys per workgroup (a multiple of 32) and the most
                             // chunks a tile can have; max_chunks == 1: a tile's keys are never split
};

// Per-wave online-softmax state for one 16-row tile. Lane (r, g) belongs to row r.
template <typename T, int DTMAX>
struct RowTile {
  typedef typename Elem<T>::Frag Frag;
  typedef typename KeyQuad<T>::Type Quad;
  static constexpr int EPF = Elem<T>::kPerFrag;
  static constexpr int NSMAX = AttnShape<T, DTMAX>::NSMAX;

  Frag qf[NSMAX];
  f32x4 acc[DTMAX];
  float m, l;

  __device__ __forceinline__ void init(const T* q_row /* null: no such row */, int head_dim, int g) {
    const int chunks = head_dim / EPF;
#pragma unroll
    for (int s = 0; s < NSMAX; ++s) {
      const int chunk = s * 4 + g;
      qf[s] = (q_row && chunk < chunks) ? tw_load_frag(q_row + chunk * EPF) : Elem<T>::zero();
    }
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m = -INFINITY;
    l = 0.f;
  }

  // One tile of 16 keys starting at position p0 (a multiple of 16).
  // t_row: position of this lane's row (-1: no such row). lo_load: keys below it are never loaded.
  __device__ __forceinline__ void key_tile(const AttnArgs& a, const int* table, int kvh, int p0, int kv_len,
                                           int t_row, int lo_load, int r, int g) {
    const T* keys = (const T*)a.keys;
    const T* values = (const T*)a.values;
    const int D = a.head_dim, P = a.page_size;
    const int chunks = D / EPF, dts = D / 16;
    // ---- S^T = K Q^T ------------------------------------------------------
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    {
      const int p = p0 + r;                       // this lane loads key p's fragments
      int page = -1;
      if (p < kv_len && p >= lo_load) page = table[p / P];
      const T* k_row = keys + (((size_t)(page < 0 ? 0 : page) * a.kv_heads + kvh) * P + p % P) * D;
#pragma unroll
      for (int st = 0; st < NSMAX; ++st) {
        const int chunk = st * 4 + g;
        if (st * 4 < chunks) {
          const Frag kf = (page >= 0 && chunk < chunks) ? tw_load_frag(k_row + chunk * EPF) : Elem<T>::zero();
          tw_mma16(s, kf, qf[st]);
        }
      }
    }
    // ---- mask, online softmax (this lane: row r, keys p0 + 4g + j) ------------
    const int lo_row = a.window > 0 ? t_row - a.window + 1 : 0;
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int p = p0 + 4 * g + j;
      const bool ok = p < kv_len && p <= t_row && p >= lo_row;
      float sc = s[j] * a.scale;
      if (a.softcap > 0.f) sc = a.softcap * tanhf(sc / a.softcap);
      s[j] = ok ? sc : -INFINITY;
      mx = fmaxf(mx, s[j]);
    }
    mx = tw_rows_max(mx);
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = tw_exp<T>(m - m_use);
    f32x4 pr;
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      pr[j] = tw_exp<T>(s[j] - m_use);
      sum += pr[j];
    }
    sum = tw_rows_sum(sum);
    l = l * alpha + sum;
    m = m_new;
    // ---- O^T += V^T P^T (this lane loads d = 16 dt + r, keys p0 + 4g .. + 3) ----
    const int pv = p0 + 4 * g;
    int vpage = -1;
    if (pv < kv_len && pv + 3 >= lo_load) vpage = table[pv / P];
    const T* v_base = values + ((size_t)(vpage < 0 ? 0 : vpage) * a.kv_heads + kvh) * D * P + pv % P;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt) {
      if (dt < dts) {
        Quad vq;
        if (vpage >= 0) {
          vq = *reinterpret_cast<const Quad*>(v_base + (size_t)(dt * 16 + r) * P);
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (pv + j >= kv_len || pv + j < lo_load) vq[j] = tw_from_float<T>(0.f);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) vq[j] = tw_from_float<T>(0.f);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[dt][j] *= alpha;
        tw_mma16_k4(acc[dt], vq, pr);
      }
    }
  }
};

// =====================================================================================
// Decode: one token per sequence. grid = (splits, kv_heads * row_tiles, n_seqs).
// =====================================================================================
template <typename T, int DTMAX>
__global__ __launch_bounds__(256) void attn_decode_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) float lds_o[3][16][DTMAX * 16 + 8];   // (rows of 32 bytes more than a multiple of 256: see tw_lds_swz4)
  __shared__ float lds_ml[3][16][2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int G = a.q_heads / a.kv_heads;
  const int row_tiles = (G + 15) / 16;
  const int kvh = blockIdx.y / row_tiles, rt = blockIdx.y % row_tiles;
  const int seq = a.seq0 + blockIdx.z;
  const int split = blockIdx.x;
  const int kv_len = a.kv_len[seq];
  const int token = a.q_start[seq];
  const int t = kv_len - 1;
  const int* table = a.block_table + (size_t)seq * a.table_stride;
  const int D = a.head_dim, dts = D / 16;

  const int hig = rt * 16 + r;                      // head within the group
  const bool row_ok = hig < G;
  const int head = kvh * G + hig;
  RowTile<T, DTMAX> tile;
  tile.init(row_ok ? (const T*)a.q + (size_t)token * a.ldq + (size_t)head * D : nullptr, D, g);

  const int lo = a.window > 0 ? max(0, t - a.window + 1) : 0;
  const int tile_lo = lo / 16, tile_hi = (kv_len + 15) / 16;     // key tiles [tile_lo, tile_hi)
  const int per_split = (tile_hi - tile_lo + a.splits - 1) / a.splits;
  const int begin = tile_lo + split * per_split;
  const int end = min(tile_hi, begin + per_split);
  for (int kt = begin + wave; kt < end; kt += 4)
    tile.key_tile(a, table, kvh, kt * 16, kv_len, row_ok ? t : -1, lo, r, g);

  // ---- merge the 4 waves (fixed order: wave 0 absorbs 1, 2, 3) -------------------
  if (wave > 0) {
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) lds_o[wave - 1][r][dt * 16 + 4 * g + j] = tile.acc[dt][j];
    if (g == 0) {
      lds_ml[wave - 1][r][0] = tile.m;
      lds_ml[wave - 1][r][1] = tile.l;
    }
  }
  __syncthreads();
  if (wave > 0) return;
  float m = tile.m, l = tile.l;
#pragma unroll
  for (int w = 0; w < 3; ++w) m = fmaxf(m, lds_ml[w][r][0]);
  const float m_use = m == -INFINITY ? 0.f : m;
  const float own = tw_exp<T>(tile.m - m_use);
  l *= own;
#pragma unroll
  for (int dt = 0; dt < DTMAX; ++dt)
#pragma unroll
    for (int j = 0; j < 4; ++j) tile.acc[dt][j] *= own;
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    const float f = tw_exp<T>(lds_ml[w][r][0] - m_use);
    l += lds_ml[w][r][1] * f;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) tile.acc[dt][j] += lds_o[w][r][dt * 16 + 4 * g + j] * f;
  }
  if (!row_ok) return;
  if (a.splits == 1) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    T* dst = (T*)a.out + (size_t)token * a.ldo + (size_t)head * D;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[dt * 16 + 4 * g + j] = tw_from_float<T>(tile.acc[dt][j] * inv);
  } else {
    const size_t slot = ((size_t)blockIdx.z * a.q_heads + head) * a.splits + split;
    float* dst = a.part_o + slot * D;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[dt * 16 + 4 * g + j] = tile.acc[dt][j];
    if (g == 0) {
      a.part_ml[slot * 2] = m;
      a.part_ml[slot * 2 + 1] = l;
    }
  }
}

// =====================================================================================
// Decode, bfloat16, pages of 8 keys or a multiple: blocks of 32 keys.
// Row i = 4a + j of the block's first (second) score tile stands for key 8a + j
// (8a + 4 + j), so lane group g ends up with the probabilities of the 8
// CONSECUTIVE keys 8g .. 8g+7: they are the B operand of one 16x16x32 MFMA per
// 16 output dims, whose A operand is a single 16-byte load of values[d][8g..8g+7].
//
// A wave keeps two blocks in registers: the loads of the next block are in flight while
// this one is computed. Loads carry no predicate: a key outside the sequence or the window
// is read from a page the block does hold (its score is then selected to -inf and its value
// to zero), and only the first and last block of a range pay for those selects.
// EXACT: head_dim == 16 * DTMAX (no per-chunk checks at all).
// =====================================================================================
template <int DTMAX>
struct KVBlock {
  static constexpr int NSMAX = AttnShape<bf16_t, DTMAX>::NSMAX;
  bf16x8 k[2][NSMAX];
  bf16x8 v[DTMAX];
};

template <bool V> struct BoolTag { static constexpr bool value = V; };

template <int DTMAX, bool EXACT>
__global__ __launch_bounds__(256) void attn_decode_bf16_kernel(AttnArgs a) {
  constexpr int NSMAX = AttnShape<bf16_t, DTMAX>::NSMAX;
  __shared__ __attribute__((aligned(16))) float lds_o[3][16][DTMAX * 16 + 8];   // (rows of 32 bytes more than a multiple of 256: see tw_lds_swz4)
  __shared__ float lds_ml[3][16][2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int G = a.q_heads / a.kv_heads;
  const int row_tiles = (G + 15) / 16;
  const int kvh = blockIdx.y / row_tiles, rt = blockIdx.y % row_tiles;
  const int seq = a.seq0 + blockIdx.z;
  const int split = blockIdx.x;
  const int kv_len = a.kv_len[seq];
  const int token = a.q_start[seq];
  const int t = kv_len - 1;
  const int* table = a.block_table + (size_t)seq * a.table_stride;
  const int D = EXACT ? DTMAX * 16 : a.head_dim, dts = D / 16, chunks = D / 8, P = a.page_size;
  const bf16_t* keys = (const bf16_t*)a.keys;
  const bf16_t* values = (const bf16_t*)a.values;

  const int hig = rt * 16 + r;
  const bool row_ok = hig < G;
  const int head = kvh * G + hig;
  bf16x8 qf[NSMAX];
  {
    const bf16_t* q_row = (const bf16_t*)a.q + (size_t)token * a.ldq + (size_t)head * D;
#pragma unroll
    for (int st = 0; st < NSMAX; ++st) {
      const int chunk = st * 4 + g;
      qf[st] = (row_ok && (EXACT || chunk < chunks)) ? tw_load_frag(q_row + chunk * 8) : Elem<bf16_t>::zero();
    }
  }
  f32x4 acc[DTMAX];
#pragma unroll
  for (int dt = 0; dt < DTMAX; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const int lo = a.window > 0 ? max(0, t - a.window + 1) : 0;
  const int blk_lo = lo / 32, blk_hi = (kv_len + 31) / 32;
  const int per_split = (blk_hi - blk_lo + a.splits - 1) / a.splits;
  const int begin = blk_lo + split * per_split;
  const int end = min(blk_hi, begin + per_split);

  // Per-lane constants of the loads. A 32-key block spans 1, 2 or 4 pages (pages of 8 keys
  // or more, powers of two); p0 is a multiple of 32, so for pages smaller than a block the
  // in-page index of a key does not depend on the block.
  const int pshift = a.page_shift, pmask = P - 1;
  const int ppb = P >= 32 ? 1 : (32 >> pshift);                    // pages per block
  const size_t head_stride = (size_t)P * D;                          // elements of one (page, kv head)
  int k_pi[2];
  unsigned k_off[2];
#pragma unroll
  for (int tile = 0; tile < 2; ++tile) {
    const int ko = 8 * (r >> 2) + 4 * tile + (r & 3);                // the key this lane's row stands for
    k_pi[tile] = P >= 32 ? 0 : (ko >> pshift);
    k_off[tile] = (unsigned)(P >= 32 ? ko : (ko & pmask)) * D + g * 8;
  }
  const int kv0 = 8 * g;                                              // this lane's 8 consecutive keys
  const int v_pi = P >= 32 ? 0 : (kv0 >> pshift);
  const unsigned v_off = (unsigned)r * P + (P >= 32 ? kv0 : (kv0 & pmask));

  // Page ids of a block are the same for every lane: scalar loads (blk is wave-uniform).
  // A page that holds no key of [lo, kv_len) may not be held at all: it is replaced by one
  // of the block that is, so that every load has an address inside the pool.
  auto issue = [&](int blk_v, KVBlock<DTMAX>& L) {
    const int blk = __builtin_amdgcn_readfirstlane(blk_v);
    const int p0 = blk * 32;
    const int first = p0 >> pshift;
    int pg[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int a0 = P >= 32 ? p0 : p0 + (i << pshift);              // first key of the block in page i
      const int a1 = P >= 32 ? p0 + 31 : a0 + P - 1;                 // last one
      pg[i] = (i < ppb && a0 < kv_len && a1 >= lo) ? table[first + i] : -1;
    }
    int safe = pg[0] >= 0 ? pg[0] : (pg[1] >= 0 ? pg[1] : (pg[2] >= 0 ? pg[2] : pg[3]));
    if (safe < 0) safe = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (pg[i] < 0) pg[i] = safe;
    auto page_of = [&](int i) { return i == 0 ? pg[0] : (i == 1 ? pg[1] : (i == 2 ? pg[2] : pg[3])); };
    const unsigned pb = P >= 32 ? (unsigned)(p0 & pmask) : 0u;      // the block's first key inside its page
#pragma unroll
    for (int tile = 0; tile < 2; ++tile) {
      const bf16_t* k_row = keys + ((size_t)page_of(k_pi[tile]) * a.kv_heads + kvh) * head_stride + pb * D + k_off[tile];
#pragma unroll
      for (int st = 0; st < NSMAX; ++st)
        L.k[tile][st] = (EXACT || st * 4 + g < chunks) ? tw_load_frag_stream(k_row + st * 32) : Elem<bf16_t>::zero();
    }
    const bf16_t* v_base = values + ((size_t)page_of(v_pi) * a.kv_heads + kvh) * head_stride + pb + v_off;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts) L.v[dt] = tw_load_frag_stream(v_base + (size_t)(dt * 16) * P);
  };

  auto compute_as = [&](int blk, KVBlock<DTMAX>& L, auto edge_tag) {
    constexpr bool EDGE = decltype(edge_tag)::value;
    const int p0 = blk * 32;
    f32x4 s[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int tile = 0; tile < 2; ++tile)
#pragma unroll
      for (int st = 0; st < NSMAX; ++st)
        if (EXACT || st * 4 < chunks) tw_mma16(s[tile], L.k[tile][st], qf[st]);
    // this lane: row r (a head), keys p0 + 8g + e, e = 4*tile + j; every cached key is at or before t
    float pr[8];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int p = p0 + 8 * g + e;
      pr[e] = (!EDGE || (p < kv_len && p >= lo)) ? s[e >> 2][e & 3] * a.scale : -INFINITY;
      mx = fmaxf(mx, pr[e]);
    }
    mx = tw_rows_max(mx);
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    float sum = 0.f;
    bf16x8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pe = __expf(pr[e] - m_use);
      sum += pe;
      pb[e] = (bf16_t)pe;
    }
    // (l is this lane's sum over its 8 keys of every block; the four lane groups of a row are added up
    // once, after the loop: the maximum, and with it every rescaling, is the row's)
    // the running maximum of a row rarely moves after the first blocks: rescale only then
    if (__any(m_new > m)) {
      const float alpha = __expf(m - m_use);
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < DTMAX; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[dt][j] *= alpha;
      m = m_new;
    }
    l += sum;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts) {
        bf16x8 vq = L.v[dt];
        if (EDGE) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int p = p0 + 8 * g + e;
            if (p >= kv_len || p < lo) vq[e] = (bf16_t)0.f;
          }
        }
        tw_mma16(acc[dt], vq, pb);
      }
  };
  auto compute = [&](int blk, KVBlock<DTMAX>& L) {
    if (blk * 32 + 32 > kv_len || blk * 32 < lo) compute_as(blk, L, BoolTag<true>());
    else compute_as(blk, L, BoolTag<false>());
  };

  {
    KVBlock<DTMAX> A, B;
    int blk = begin + wave;                                     // this wave's blocks: blk, blk + 4, ...
    if (blk < end) {
      issue(blk, A);
      while (blk + 8 < end) {                                   // blocks blk + 4 and blk + 8 exist
        issue(blk + 4, B);
        compute(blk, A);
        issue(blk + 8, A);
        compute(blk + 4, B);
        blk += 8;
      }
      if (blk + 4 < end) {
        issue(blk + 4, B);
        compute(blk, A);
        compute(blk + 4, B);
      } else {
        compute(blk, A);
      }
    }
  }

  l = tw_rows_sum(l);
  // ---- merge the 4 waves (fixed order: wave 0 absorbs 1, 2, 3) -------------------
  if (wave > 0) {
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) lds_o[wave - 1][r][dt * 16 + 4 * g + j] = acc[dt][j];
    if (g == 0) {
      lds_ml[wave - 1][r][0] = m;
      lds_ml[wave - 1][r][1] = l;
    }
  }
  __syncthreads();
  if (wave > 0) return;
  float m_all = m;
#pragma unroll
  for (int w = 0; w < 3; ++w) m_all = fmaxf(m_all, lds_ml[w][r][0]);
  const float m_use = m_all == -INFINITY ? 0.f : m_all;
  const float own = __expf(m - m_use);
  l *= own;
#pragma unroll
  for (int dt = 0; dt < DTMAX; ++dt)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[dt][j] *= own;
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    const float f = __expf(lds_ml[w][r][0] - m_use);
    l += lds_ml[w][r][1] * f;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[dt][j] += lds_o[w][r][dt * 16 + 4 * g + j] * f;
  }
  if (!row_ok) return;
  if (a.splits == 1) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    bf16_t* dst = (bf16_t*)a.out + (size_t)token * a.ldo + (size_t)head * D;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[dt * 16 + 4 * g + j] = (bf16_t)(acc[dt][j] * inv);
  } else {
    const size_t slot = ((size_t)blockIdx.z * a.q_heads + head) * a.splits + split;
    float* dst = a.part_o + slot * D;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[dt * 16 + 4 * g + j] = acc[dt][j];
    if (g == 0) {
      a.part_ml[slot * 2] = m_all;
      a.part_ml[slot * 2 + 1] = l;
    }
  }
}

// Merge the splits of one (sequence, head): grid = (q_heads, n_seqs). Thread (d, c)
// sums the splits c, c + C, ... of output dim d; the C partial sums are then
// added in a fixed order, so the result does not depend on timing.
#define TW_REDUCE_THREADS 256
template <typename T>
__global__ __launch_bounds__(TW_REDUCE_THREADS) void attn_decode_reduce_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ q_start,
    int seq0, T* out, long ldo, int q_heads, int head_dim, int splits) {
  __shared__ float s_w[64];                    // weight of each split: exp(m_s - m)
  __shared__ float s_acc[TW_REDUCE_THREADS];
  __shared__ float s_l;
  const int head = blockIdx.x, local = blockIdx.y, tid = threadIdx.x;
  const size_t slot0 = ((size_t)local * q_heads + head) * splits;
  const int cols = TW_REDUCE_THREADS / head_dim > 0 ? TW_REDUCE_THREADS / head_dim : 1;   // head_dim <= 256
  const int d = tid % head_dim, c = tid / head_dim;
  // The first 8 partial outputs of this thread are on their way while the weights are formed
  // (the kernel's time is a chain of memory latencies).
  const int token = q_start[seq0 + local];
  float po[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int sp = c + i * cols;
    po[i] = (c < cols && sp < splits) ? part_o[(slot0 + sp) * head_dim + d] : 0.f;
  }
  if (tid < 64) {
    const float mine = tid < splits ? part_ml[(slot0 + tid) * 2] : -INFINITY;
    const float m = tw_wave_max(mine);
    const float m_use = m == -INFINITY ? 0.f : m;
    const float w = tid < splits ? expf(mine - m_use) : 0.f;
    s_w[tid] = w;
    const float lw = tid < splits ? part_ml[(slot0 + tid) * 2 + 1] * w : 0.f;
    // fixed-order sum over the splits
    float l = 0.f;
    for (int i = 0; i < 64; ++i) l += __shfl(lw, i, TW_WAVE);
    if (tid == 0) s_l = l;
  }
  __syncthreads();
  float o = 0.f;
  if (c < cols) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int sp = c + i * cols;
      if (sp < splits) o += po[i] * s_w[sp];
    }
    for (int sp = c + 8 * cols; sp < splits; sp += cols) o += part_o[(slot0 + sp) * head_dim + d] * s_w[sp];
  }
  s_acc[tid] = o;
  __syncthreads();
  if (tid < head_dim) {
    float total = 0.f;
    for (int i = 0; i < cols; ++i) total += s_acc[i * head_dim + tid];
    const float l = s_l;
    out[(size_t)token * ldo + (size_t)head * head_dim + tid] = tw_from_float<T>(l > 0.f ? total / l : 0.f);
  }
}

// =====================================================================================
// Prefill: q_len tokens of a sequence. grid = (row tiles / 4, kv_heads, n_seqs);
// each of the 4 waves of a workgroup takes one tile of 16 (token, head) rows.
// =====================================================================================
template <typename T, int DTMAX>
__global__ __launch_bounds__(256) void attn_prefill_kernel(AttnArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int G = a.q_heads / a.kv_heads;
  const int kvh = blockIdx.y;
  const int seq = a.seq0 + blockIdx.z;
  const int kv_len = a.kv_len[seq];
  const int token0 = a.q_start[seq];
  const int q_len = a.q_start[seq + 1] - token0;
  const int rows = q_len * G;
  const int row0 = (blockIdx.x * 4 + wave) * 16;
  if (row0 >= rows) return;
  const int* table = a.block_table + (size_t)seq * a.table_stride;
  const int D = a.head_dim, dts = D / 16;

  const int row = row0 + r;
  const bool row_ok = row < rows;
  const int tok = row / G, hig = row % G;            // token within the portion, head within the group
  const int head = kvh * G + hig;
  const int first_pos = kv_len - q_len;              // position of the portion's first token
  const int t_row = row_ok ? first_pos + tok : -1;
  RowTile<T, DTMAX> tile;
  tile.init(row_ok ? (const T*)a.q + (size_t)(token0 + tok) * a.ldq + (size_t)head * D : nullptr, D, g);

  const int t_min = first_pos + row0 / G;
  const int t_max = first_pos + min(rows - 1, row0 + 15) / G;
  const int lo = a.window > 0 ? max(0, t_min - a.window + 1) : 0;
  for (int kt = lo / 16; kt * 16 <= t_max; ++kt)
    tile.key_tile(a, table, kvh, kt * 16, kv_len, t_row, lo, r, g);

  if (!row_ok) return;
  const float inv = tile.l > 0.f ? 1.f / tile.l : 0.f;
  T* dst = (T*)a.out + (size_t)(token0 + tok) * a.ldo + (size_t)head * D;
#pragma unroll
  for (int dt = 0; dt < DTMAX; ++dt)
    if (dt < dts)
#pragma unroll
      for (int j = 0; j < 4; ++j) dst[dt * 16 + 4 * g + j] = tw_from_float<T>(tile.acc[dt][j] * inv);
}

// =====================================================================================
// Prefill, bfloat16, pages of 8 keys or a power of two above: a workgroup of 4
// waves owns 128 (or 64) consecutive (token, head) rows of one kv head, 32 (16) per wave. The
// keys and values of each 32-key block are copied ONCE per workgroup into LDS
// (keys outside the sequence as zeros) while the block before is computed; every
// K or V fragment a wave reads from LDS serves both of its 16-row tiles.
// Key/row layout inside a block as in the decode kernel above.
// =====================================================================================
#define TW_PF_VROW 64                       /* LDS bytes per value row (32 keys; the 16-byte pieces of row d lie at piece ^ tw_lds_swz4(d)) */
#define TW_PF_SLACK 8.f                     /* how far, in powers of two, a score may exceed the reference of its row before that is moved */
#define TW_PF_STAGES 3                      /* blocks in LDS: the one whose probabilities are formed, the one whose scores are, the one being written */


// EXACT: head_dim == 16 * DTMAX, so every loop over the head has compile-time bounds (with run-time
// bounds the compiler indexes the accumulators dynamically, several instructions per MFMA).
template <int DTMAX, bool EXACT, int RT>
__global__ __launch_bounds__(256) void attn_prefill_bf16_kernel(AttnArgs a) {
  constexpr int TR = 64 * RT;                           // rows of a workgroup's tile: RT tiles of 16 per wave
  constexpr int NSMAX = AttnShape<bf16_t, DTMAX>::NSMAX;
  constexpr int KROW = DTMAX * 32 + 32;                 // LDS bytes per key row, padded: 32 * an odd number (see tw_lds_swz4)
  static_assert(DTMAX % 2 == 0, "the padding of a key row assumes an even number of 32-byte pieces");
  constexpr int KSTAGE = 32 * KROW, VSTAGE = DTMAX * 16 * TW_PF_VROW;
  constexpr int KPIECES = (32 * DTMAX * 2 + 255) / 256;  // 16-byte pieces per thread per block
  constexpr int VPIECES = (DTMAX * 16 * 4 + 255) / 256;
  constexpr int CH = DTMAX * 2;                          // 16-byte chunks per key row of this size class
  // every thread's every piece is part of the block (then the copies to LDS carry no lane mask, which costs
  // a dozen scalar instructions a piece)
  constexpr bool ALL_USED = EXACT && (32 * CH) % 256 == 0 && (DTMAX * 16 * 4) % 256 == 0;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* lds_k = lds;
  char* lds_v = lds + TW_PF_STAGES * KSTAGE;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // the same for the wave's lanes: what follows from it stays scalar
  const int r = lane & 15, g = lane >> 4;
  const int G = a.q_heads / a.kv_heads;
  // Which tile this workgroup takes. Tiles are ranked by the keys they see (most first: rank =
  // tile-from-the-end major, then kv head and sequence). Workgroups are handed to the 8 XCDs in
  // turn and, within an XCD, to its 32 CUs in turn; while all of them are resident (at most two
  // per CU), a CU's second workgroup is given the rank that evens out the sum of the two, and the
  // CUs that get one workgroup the heaviest ranks. With more workgroups than that, heaviest first.
  int rank;
  {
    const int total = gridDim.x, b = blockIdx.x, xcd = b & 7, j = b >> 3;
    const int n = (total - xcd + 7) >> 3;                       // workgroups of this XCD
    constexpr int C = 32;
    int r = j;
    if (n > C && n <= 2 * C) {
      const int paired = n - C, single = C - paired;
      if (j < paired) r = single + j;                           // first of a pair
      else if (j < C) r = j - paired;                           // alone on its CU: the heaviest
      else r = n - 1 - (j - C);                                 // second of a pair: mirrors the first
    }
    rank = r * 8 + xcd;
    if (rank >= total) rank = b;                                 // (uneven XCD shares: keep every tile covered)
  }
  // (the divisions run on the vector unit; what they give is the same for every lane, and saying so
  // keeps the block-table lookups and page addresses of the loop below on the scalar unit)
  const int chunk = __builtin_amdgcn_readfirstlane(rank % a.max_chunks);
  rank /= a.max_chunks;
  const int per_tile = a.kv_heads * a.n_seqs;
  const int tile_from_end = __builtin_amdgcn_readfirstlane(rank / per_tile), sub = rank % per_tile;
  const int kvh = __builtin_amdgcn_readfirstlane(sub % a.kv_heads);
  const int seq = __builtin_amdgcn_readfirstlane(a.seq0 + sub / a.kv_heads);
  const int kv_len = a.kv_len[seq];
  const int token0 = a.q_start[seq];
  const int q_len = a.q_start[seq + 1] - token0;
  const int rows = q_len * G;
  const int n_tiles = (rows + TR - 1) / TR;
  const int tile_idx = a.max_tiles - 1 - tile_from_end;         // counted from the longest sequence's last tile
  if (tile_idx < 0 || tile_idx >= n_tiles) return;
  const int wg_row0 = tile_idx * TR;
  const int* table = a.block_table + (size_t)seq * a.table_stride;
  const int D = EXACT ? DTMAX * 16 : a.head_dim, dts = D / 16, chunks = D / 8, P = a.page_size;
  const int pshift = a.page_shift, pmask = P - 1;
  const unsigned head_stride = (unsigned)P * D;
  const bf16_t* keys = (const bf16_t*)a.keys;
  const bf16_t* values = (const bf16_t*)a.values;
  const int first_pos = kv_len - q_len;
  const bool whole_chunks = EXACT || (chunks & 3) == 0;  // head_dim a multiple of 32: no partial MFMA step
  const float c2 = a.scale * 1.44269504088896340736f;    // scores are kept in the log2 domain

  // ---- this wave's two row tiles -----------------------------------------------
  bf16x8 qf[RT][NSMAX];
  int t_row[RT], tok[RT], head[RT];
  bool row_ok[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = wg_row0 + wave * 16 * RT + rt * 16 + r;
    row_ok[rt] = row < rows;
    tok[rt] = row / G;
    head[rt] = kvh * G + row % G;
    // (a row past the end stands in for the last token with a query of zeros: it sees what the wave's
    // other rows see, needs no mask of its own, and is never stored)
    t_row[rt] = first_pos + (row_ok[rt] ? tok[rt] : (rows - 1) / G);
    const bf16_t* q_row = (const bf16_t*)a.q + (size_t)(token0 + tok[rt]) * a.ldq + (size_t)head[rt] * D;
#pragma unroll
    for (int st = 0; st < NSMAX; ++st) {
      const int chunk = st * 4 + g;
      qf[rt][st] = (row_ok[rt] && (EXACT || chunk < chunks)) ? tw_load_frag(q_row + chunk * 8) : Elem<bf16_t>::zero();
    }
  }
  f32x4 acc[RT][DTMAX];
  float m[RT], l[RT];
  f32x4 l_mma[RT];                                           // row sums that the matrix unit forms (the hand-ordered iterations)
  float m_use[RT], m_thr[RT];                                // what the exponentials subtract (0 while m is -inf); the score above which m moves
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    m[rt] = -INFINITY;
    m_use[rt] = 0.f;
    m_thr[rt] = -INFINITY;
    l[rt] = 0.f;
    l_mma[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt) acc[rt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- the workgroup's key range ------------------------------------------------
  const int t_min = first_pos + wg_row0 / G;
  const int t_max = first_pos + min(rows - 1, wg_row0 + TR - 1) / G;
  const int lo = a.window > 0 ? max(0, t_min - a.window + 1) : 0;       // keys below are never loaded
  // The tile's key blocks, and the share of them this workgroup takes. A tile split into several
  // chunks leaves float32 partial results (running maximum, sum, output) that a second kernel merges.
  const int tile_begin = lo / 32, tile_end = t_max / 32 + 1;
  const int chunk_blocks = a.max_chunks > 1 ? a.kv_chunk / 32 : tile_end - tile_begin;
  const int n_chunks = (tile_end - tile_begin + chunk_blocks - 1) / chunk_blocks;
  if (chunk >= n_chunks) return;
  const int blk_begin = tile_begin + chunk * chunk_blocks, blk_end = min(tile_end, blk_begin + chunk_blocks);
  const int wave_t_max = first_pos + min(rows - 1, wg_row0 + wave * 16 * RT + 16 * RT - 1) / G;
  const int wave_t_min = first_pos + min(rows - 1, wg_row0 + wave * 16 * RT) / G;
  const bool wave_live = wg_row0 + wave * 16 * RT < rows;
  const int wave_lo_max = a.window > 0 ? wave_t_max - a.window + 1 : 0;  // largest lower bound among the wave's rows

  // This thread's share of a block, fixed for the whole loop: K piece i is 16 bytes
  // (chunk k_chunk) of key k_key; V piece i is keys 8*v_oct .. +7 of output dim v_d.
  bf16x8 kreg[KPIECES], vreg[VPIECES];
  int k_key[KPIECES], k_goff[KPIECES], k_loff[KPIECES], k_slot[KPIECES];
  int v_oct[VPIECES], v_goff[VPIECES], v_loff[VPIECES], v_slot[VPIECES];
  bool k_use[KPIECES], v_use[VPIECES];
#pragma unroll
  for (int i = 0; i < KPIECES; ++i) {
    const int q = tid + i * 256, key = q / CH, chunk = q % CH;
    k_use[i] = key < 32 && chunk < chunks;
    k_key[i] = key;
    const int key_c = min(key, 31), chunk_c = min(chunk, chunks - 1);   // an unused piece loads a used one's bytes
    k_slot[i] = P >= 32 ? 0 : (key_c >> pshift);           // which of the block's pages
    k_goff[i] = (P >= 32 ? key_c : (key_c & pmask)) * D + chunk_c * 8;
    // key k lies in LDS row (k / 8 % 4) * 4 + k % 4 + 16 * (k / 4 % 2): the 16 keys whose scores one MFMA
    // forms (k % 8 < 4, or >= 4) are 16 consecutive rows, which with the row length KROW a fragment read
    // finds in 16 different 16-byte columns of the banks (see tw_lds_swz4)
    k_loff[i] = (((key >> 3) & 3) * 4 + (key & 3) + 16 * ((key >> 2) & 1)) * KROW + chunk * 16;
  }
#pragma unroll
  for (int i = 0; i < VPIECES; ++i) {
    const int q = tid + i * 256, d = q >> 2, oct = q & 3;
    v_use[i] = d < D;
    v_oct[i] = oct;
    v_slot[i] = P >= 32 ? 0 : ((8 * oct) >> pshift);
    v_goff[i] = min(d, D - 1) * P + (P >= 32 ? 8 * oct : ((8 * oct) & pmask));
    v_loff[i] = d * TW_PF_VROW + ((oct ^ tw_lds_swz4(d)) * 16);
  }
  // global -> registers. Loads carry no predicate: a page of the block that holds no key of
  // [lo, kv_len) may not be held at all and is replaced by one of the block that is, so every
  // address lies inside the pool; what such keys hold never counts (their scores are selected
  // to -inf) except in the PV product, so their VALUES are made zero here, in the rare block
  // that crosses the end of the sequence or the start of the window.
  // Each lane looks up the pages of its own pieces in the block table, one block ahead of the
  // fetch (all four waves doing the same table arithmetic on the CU's one scalar unit was what
  // bounded this kernel).
  int k_pg[KPIECES], v_pg[VPIECES];
  auto lookup = [&](int blk_v) {
    const int blk = __builtin_amdgcn_readfirstlane(min(blk_v, blk_end - 1));
    const int p0 = blk * 32;
    const int* entry = table + (p0 >> pshift);
    if (p0 >= lo && p0 + 32 <= kv_len) {                     // every key of the block counts: the common case
#pragma unroll
      for (int i = 0; i < KPIECES; ++i) k_pg[i] = entry[k_slot[i]];
#pragma unroll
      for (int i = 0; i < VPIECES; ++i) v_pg[i] = entry[v_slot[i]];
    } else {
      const int safe = P >= 32 ? 0 : ((max(lo, p0) - p0) >> pshift);   // a page of the block that is held
      auto held = [&](int slot) {
        const int a0 = P >= 32 ? p0 : p0 + (slot << pshift);
        const int a1 = P >= 32 ? p0 + 31 : a0 + P - 1;
        return (a0 < kv_len && a1 >= lo) ? slot : safe;
      };
#pragma unroll
      for (int i = 0; i < KPIECES; ++i) k_pg[i] = entry[held(k_slot[i])];
#pragma unroll
      for (int i = 0; i < VPIECES; ++i) v_pg[i] = entry[held(v_slot[i])];
    }
  };
  // Where this lane's pieces lie in page 0 of its kv head: an address is that plus page * (bytes of a page)
  // plus where the block starts inside its page, one 32 x 32 -> 64 bit multiply-add and one 64-bit add a
  // piece (the launcher checks that a page's bytes fit 32 bits; page numbers are not negative).
  const unsigned page_bytes = (unsigned)a.kv_heads * head_stride * 2u;
  const char* k_at[KPIECES];
  const char* v_at[VPIECES];
#pragma unroll
  for (int i = 0; i < KPIECES; ++i) k_at[i] = (const char*)keys + ((size_t)kvh * head_stride + k_goff[i]) * 2;
#pragma unroll
  for (int i = 0; i < VPIECES; ++i) v_at[i] = (const char*)values + ((size_t)kvh * head_stride + v_goff[i]) * 2;
  auto fetch = [&](int blk_v) {                              // (after lookup of the same block)
    const int blk = __builtin_amdgcn_readfirstlane(blk_v);
    const int p0 = blk * 32;
    const unsigned in_page = P >= 32 ? (unsigned)(p0 & pmask) : 0u;   // where the block starts inside its page
    const unsigned k_in = in_page * (unsigned)D * 2u, v_in = in_page * 2u;
#pragma unroll
    for (int i = 0; i < KPIECES; ++i)
      kreg[i] = tw_load_frag((const bf16_t*)(k_at[i] + ((uint64_t)(unsigned)k_pg[i] * page_bytes + k_in)));
#pragma unroll
    for (int i = 0; i < VPIECES; ++i)
      vreg[i] = tw_load_frag((const bf16_t*)(v_at[i] + ((uint64_t)(unsigned)v_pg[i] * page_bytes + v_in)));
    if (p0 + 32 > kv_len || p0 < lo) {
#pragma unroll
      for (int i = 0; i < VPIECES; ++i) {
        const int p = p0 + 8 * v_oct[i];
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (p + e >= kv_len || p + e < lo) vreg[i][e] = (bf16_t)0.f;
      }
    }
  };
  // (one piece at a time, for a block every key of which counts: i < KPIECES is K piece i, the others are V's)
  auto lookup_piece = [&](int i, const int* entry) {
    if (i < KPIECES) k_pg[i] = entry[k_slot[i]];
    else v_pg[i - KPIECES] = entry[v_slot[i - KPIECES]];
  };
  auto fetch_piece = [&](int i, unsigned k_in, unsigned v_in) {
    if (i < KPIECES) kreg[i] = tw_load_frag((const bf16_t*)(k_at[i] + ((uint64_t)(unsigned)k_pg[i] * page_bytes + k_in)));
    else vreg[i - KPIECES] = tw_load_frag((const bf16_t*)(v_at[i - KPIECES] + ((uint64_t)(unsigned)v_pg[i - KPIECES] * page_bytes + v_in)));
  };
  auto stash_piece = [&](int i, int buf) {
    if (i < KPIECES) {
      if (ALL_USED || k_use[i]) *reinterpret_cast<bf16x8*>(lds_k + buf * KSTAGE + k_loff[i]) = kreg[i];
    } else if (ALL_USED || v_use[i - KPIECES]) {
      *reinterpret_cast<bf16x8*>(lds_v + buf * VSTAGE + v_loff[i - KPIECES]) = vreg[i - KPIECES];
    }
  };
  auto stash = [&](int buf) {                                // registers -> LDS
#pragma unroll
    for (int i = 0; i < KPIECES; ++i)
      if (ALL_USED || k_use[i]) *reinterpret_cast<bf16x8*>(lds_k + buf * KSTAGE + k_loff[i]) = kreg[i];
#pragma unroll
    for (int i = 0; i < VPIECES; ++i)
      if (ALL_USED || v_use[i]) *reinterpret_cast<bf16x8*>(lds_v + buf * VSTAGE + v_loff[i]) = vreg[i];
  };

  // LDS addresses of this lane's fragments in stage 0
  const char* k_frag[2];
#pragma unroll
  for (int tile = 0; tile < 2; ++tile)
    k_frag[tile] = lds_k + (16 * tile + r) * KROW + g * 16;   // (lane r's key of the tile: 8 (r / 4) + 4 tile + r % 4)
  const char* v_frag = lds_v + r * TW_PF_VROW + ((g ^ tw_lds_swz4(r)) * 16);

  // A block is worked on in two steps, one iteration apart: its SCORES, S^T = K Q^T, and, an iteration
  // later, the softmax of those and the PV products. In an iteration the scores of block b + 1 (matrix
  // unit) and the softmax of block b (vector unit) do not depend on each other, so one wave keeps both
  // units busy; with both in one step the two took turns.
  // edge: some key of the block is hidden from some row of the wave; only then are scores masked.
  // (with the largest heads and 128-row tiles the two steps stay in one iteration: there are not the
  // registers for two blocks' scores beside the output)
  constexpr bool PIPELINED = DTMAX * RT <= 16;
  // the K fragments of a block (stage buf), and the scores of one row tile against them
  auto k_fragments = [&](int buf, bf16x8 (&kf)[2][NSMAX]) {
#pragma unroll
    for (int tile = 0; tile < 2; ++tile) {
      const char* base = k_frag[tile] + buf * KSTAGE;
#pragma unroll
      for (int st = 0; st < NSMAX; ++st)
        if (EXACT || st * 4 < chunks) {
          kf[tile][st] = *reinterpret_cast<const bf16x8*>(base + st * 64);
          if (!whole_chunks && st * 4 + g >= chunks) kf[tile][st] = Elem<bf16_t>::zero();
        }
    }
  };
  auto scores_of = [&](int rt, const bf16x8 (&kf)[2][NSMAX], f32x4 (&s)[RT][2]) {
#pragma unroll
    for (int tile = 0; tile < 2; ++tile) s[rt][tile] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < NSMAX; ++st)
      if (EXACT || st * 4 < chunks)
#pragma unroll
        for (int tile = 0; tile < 2; ++tile) tw_mma16(s[rt][tile], kf[tile][st], qf[rt][st]);
  };
  auto scores = [&](int blk, int buf, bool edge, f32x4 (&s)[RT][2]) {
    const int p0 = blk * 32;
    bf16x8 kf[2][NSMAX];
    k_fragments(buf, kf);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) scores_of(rt, kf, s);
    if (edge) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int lo_row = a.window > 0 ? t_row[rt] - a.window + 1 : 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int p = p0 + 8 * g + e;
          if (!(p <= t_row[rt] && p >= lo_row && p < kv_len)) s[rt][e >> 2][e & 3] = -INFINITY;
        }
      }
    }
  };
  // The softmax of a row tile's scores, in three parts.
  // m, in the scaled log2 domain (score * c2, c2 > 0), is the REFERENCE the exponentials are taken
  // against: the row's largest score when it was last moved, and it is moved only when a score exceeds
  // it by more than TW_PF_SLACK (then the running sum and output are rescaled). Until then probabilities
  // may be as large as 2^TW_PF_SLACK instead of 1; sum and output are relative to the same reference, so
  // their quotient is what it would be against the true maximum, and float32 and bfloat16 keep their
  // relative precision at that size. The reference moves in the first block of a row tile and hardly
  // ever again, so the test for it is made as cheap as it can be: each lane compares the largest of ITS
  // eight scores with the row's threshold, (m + slack) / c2, and only if some lane of the wave is above
  // it are the row's maximum formed across lanes, the reference moved and sum and output rescaled (which
  // makes the other waves of the workgroup wait at the next barrier).
  auto max3 = [](float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
  };
  auto max2 = [](float a, float b) {
    float d;
    asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
  };
  auto move_reference = [&](const float (&mx)[RT]) {        // mx: the largest of this lane's scores, per row tile
    bool above = false;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) above |= mx[rt] > m_thr[rt];
    if (__any(above)) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const float cand = tw_rows_max(mx[rt]) * c2;
        const float m_new = cand > m[rt] + TW_PF_SLACK ? cand : m[rt];
        const float use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m[rt] - use);   // (1 exactly for a row whose reference stays)
        l[rt] *= alpha;
        if constexpr (EXACT && PIPELINED) l_mma[rt] *= alpha;
        m[rt] = m_new;
        m_use[rt] = use;
        m_thr[rt] = (m_new + TW_PF_SLACK) / c2;
        // Where the output fits the vector registers (the kernels that work on two blocks at a time) it
        // is scaled as it stands. In the kernels with the largest heads it lives in accumulation registers,
        // which only MFMAs and moves can name: written as plain multiplications, the compiler moves all
        // of it into vector registers at the top of EVERY iteration, for the sake of this branch that is
        // hardly ever taken; as opaque code the moves stay in here.
#pragma unroll
        for (int dt = 0; dt < DTMAX; ++dt) {
          if constexpr (PIPELINED) {
            acc[rt][dt] *= alpha;
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float o = acc[rt][dt][j], t;
              asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 1\n\tv_accvgpr_write_b32 %0, %1"
                           : "+a"(o), "=&v"(t)
                           : "v"(alpha));
              acc[rt][dt][j] = o;
            }
          }
        }
      }
    }
  };
  auto reference = [&](const f32x4 (&s)[RT][2]) {
    float mx[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      mx[rt] = max3(s[rt][0][0], s[rt][0][1], s[rt][0][2]);
      mx[rt] = max3(mx[rt], s[rt][0][3], s[rt][1][0]);
      mx[rt] = max3(mx[rt], s[rt][1][1], s[rt][1][2]);
      mx[rt] = max2(mx[rt], s[rt][1][3]);
    }
    move_reference(mx);
  };
  auto probabilities = [&](int rt, const f32x4 (&s)[RT][2], bf16x8& pb) {
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pe = __builtin_amdgcn_exp2f(fmaf(s[rt][e >> 2][e & 3], c2, -m_use[rt]));
      sum = e == 0 ? pe : sum + pe;
      pb[e] = (bf16_t)pe;
    }
    // l is this LANE's sum (its 8 keys of every block); the four lane groups of a row are added up
    // once, after the loop
    l[rt] += sum;
  };
  auto v_fragments = [&](int buf, bf16x8 (&vf)[DTMAX]) {
    const char* vbase = v_frag + buf * VSTAGE;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts) vf[dt] = *reinterpret_cast<const bf16x8*>(vbase + dt * 16 * TW_PF_VROW);
  };
  auto products = [&](int rt, const bf16x8 (&vf)[DTMAX], const bf16x8& pb) {
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts) tw_mma16(acc[rt][dt], vf[dt], pb);
  };
  // softmax and PV products of a block whose scores are there and have been held against the reference
  auto finish = [&](int buf, f32x4 (&s)[RT][2]) {
    bf16x8 vf[DTMAX];
    v_fragments(buf, vf);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      bf16x8 pb;
      probabilities(rt, s, pb);
      products(rt, vf, pb);
    }
  };
  // Both steps in one stretch of code without a branch: the scores of the next block (stage buf1, into
  // s_next; every row sees every key of it), softmax and products of block blk (scores in s, stage buf),
  // and at the end the test of the new scores against the reference. The scheduler is asked to issue the
  // MFMAs one by one between the vector instructions they do not depend on (a wave issues in order, and
  // MFMAs issued in a row keep it from issuing anything else until the last has been taken): the new
  // scores between the first row tile's exponentials, a row tile's products between the next one's
  // exponentials, the last products between the maxima of the new scores.
  auto finish_and_score = [&](int buf, int buf1, f32x4 (&s)[RT][2], f32x4 (&s_next)[RT][2]) {
    bf16x8 kf[2][NSMAX], vf[DTMAX];
    k_fragments(buf1, kf);
    v_fragments(buf, vf);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) scores_of(rt, kf, s_next);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      bf16x8 pb;
      probabilities(rt, s, pb);
      products(rt, vf, pb);
    }
#pragma unroll
    for (int i = 0; i < 2 * NSMAX * RT; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4 / RT, 0);
    }
#pragma unroll
    for (int rt = 1; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < DTMAX; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      }
#pragma unroll
    for (int i = 0; i < DTMAX; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 1, 0);
    }
    reference(s_next);
  };
  // The same iteration in an order set by hand, for head sizes whose loops have compile-time bounds, with
  // the copies that end an iteration inside it (blocks blk + 3 and blk + 4, where they are blocks of this
  // workgroup, must be ones every key of which counts: no masking of V, no page of the table left out).
  // One SLOT is one MFMA followed by the few other instructions that share its time: at most MPS
  // memory operations (the other K fragments of the next block; the writes of block blk + 2 to LDS; the
  // loads of block blk + 3; this block's V fragments, each a few slots before its products; the page
  // numbers of block blk + 4), a share of the exponentials, and, beside the products, the maxima of the
  // new scores. Nothing crosses a slot's end. The MFMAs come in the order scores (fragment by fragment,
  // each for every row tile), products (fragment by fragment, each for every row tile: a fragment lives
  // in registers for a few slots only), sums; every exponential is in a slot before the first product.
  // The sums of the probabilities are formed by the matrix unit too, as one more product a row tile
  // (ones x P, of the probabilities as rounded for the products): the vector unit is what bounds this
  // loop, and eight additions a row tile cost it twice the time the MFMA costs the matrix unit.
  constexpr int KF_AHEAD = 2 * NSMAX < 4 ? 2 * NSMAX : 4;
  auto ordered_iteration = [&](int blk, int buf, int buf1, int buf2, f32x4 (&s)[RT][2], f32x4 (&s_next)[RT][2],
                               bf16x8 (&ahead)[KF_AHEAD]) {
    constexpr int NQK = 2 * NSMAX * RT, NPV = DTMAX * RT, NSLOT = NQK + NPV + RT;
    constexpr int NKF = 2 * NSMAX, NP = KPIECES + VPIECES;
    constexpr int NMEM = NKF + DTMAX + 3 * NP, MPS = (NMEM + NSLOT - 1) / NSLOT;
    constexpr int VF_FIRST = NKF - KF_AHEAD + 2 * NP;       // V fragment dt is memory operation VF_FIRST + dt
    constexpr int BARRIER_SLOT = (VF_FIRST + DTMAX + NP - 1) / MPS;   // the slot of the last operation before the barrier
    constexpr int NPROB = 8 * RT, P_AHEAD = 2, P_SPAN = NQK - 1;
    constexpr int NMX = 4 * RT;
    static_assert(VF_FIRST / MPS + 2 <= NQK, "the first V fragment is read two slots before its product");
    static_assert(BARRIER_SLOT < NSLOT - 1);
    static_assert(P_AHEAD < NPROB && P_SPAN >= 1);
    bf16x8 kf[NKF], vf[DTMAX], pb[RT], ones;
    float mx[RT];
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (bf16_t)1.f;
    const int fetch_blk = __builtin_amdgcn_readfirstlane(min(blk + 3, blk_end - 1));
    const int lookup_blk = __builtin_amdgcn_readfirstlane(min(blk + 4, blk_end - 1));
    const unsigned in_page = P >= 32 ? (unsigned)((fetch_blk * 32) & pmask) : 0u;
    const unsigned k_in = in_page * (unsigned)D * 2u, v_in = in_page * 2u;
    const int* entry = table + ((lookup_blk * 32) >> pshift);
    const char* kbase = k_frag[0] + buf1 * KSTAGE;           // (tile 1's fragments lie 16 rows further)
    const char* kbase_next = k_frag[0] + buf2 * KSTAGE;
    const char* vbase = v_frag + buf * VSTAGE;
    auto k_fragment = [&](auto& to, const char* base, int k) {   // k = 2 * step + tile
      to[k] = *reinterpret_cast<const bf16x8*>(base + (k & 1) * 16 * KROW + (k >> 1) * 64);
    };
    auto memory_operation = [&](int q) {
      if (q < NKF - KF_AHEAD) return k_fragment(kf, kbase, q + KF_AHEAD);
      q -= NKF - KF_AHEAD;
      if (q < NP) return stash_piece(q, buf2);
      q -= NP;
      if (q < NP) return fetch_piece(q, k_in, v_in);
      q -= NP;
      if (q < DTMAX) { vf[q] = *reinterpret_cast<const bf16x8*>(vbase + q * 16 * TW_PF_VROW); return; }
      q -= DTMAX;
      if (q < NP) return lookup_piece(q, entry);
      k_fragment(ahead, kbase_next, q - NP);                  // (behind the barrier: the block after the next)
    };
    // (the empty statements hold an exponential in its slot: its input is taken there and no earlier, its
    // rounded pair of results is there and no later; the compiler gathered them where they cost most)
    float p_odd;
    u32x4 pw[RT];
    auto exponential = [&](int j) {
      const int rt = j >> 3, e = j & 7;
      float x = s[rt][e >> 2][e & 3];
      asm volatile("" : "+v"(x));
      const float pe = __builtin_amdgcn_exp2f(fmaf(x, c2, -m_use[rt]));
      if ((e & 1) == 0) {
        p_odd = pe;
      } else {
        const bf16x2 two = {(bf16_t)p_odd, (bf16_t)pe};
        unsigned word = __builtin_bit_cast(unsigned, two);
        asm volatile("" : "+v"(word));
        pw[rt][e >> 1] = word;
        if (e == 7) pb[rt] = __builtin_bit_cast(bf16x8, pw[rt]);
      }
    };
    auto maximum = [&](int k) {
      const int rt = k >> 2;
      const f32x4 &lo4 = s_next[rt][0], &hi4 = s_next[rt][1];
      if ((k & 3) == 0) mx[rt] = max3(lo4[0], lo4[1], lo4[2]);
      else if ((k & 3) == 1) mx[rt] = max3(mx[rt], lo4[3], hi4[0]);
      else if ((k & 3) == 2) mx[rt] = max3(mx[rt], hi4[1], hi4[2]);
      else mx[rt] = max2(mx[rt], hi4[3]);
    };
#pragma unroll
    for (int k = 0; k < KF_AHEAD; ++k) kf[k] = ahead[k];     // (read behind the barrier of the iteration before)
#pragma unroll
    for (int j = 0; j < P_AHEAD; ++j) exponential(j);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int slot = 0; slot < NSLOT; ++slot) {
      if (slot < NQK) {
        const int k = slot / RT, rt = slot % RT, tile = k & 1, st = k >> 1;
        if (st == 0) s_next[rt][tile] = f32x4{0.f, 0.f, 0.f, 0.f};
        tw_mma16(s_next[rt][tile], kf[k], qf[rt][st]);
      } else if (slot < NQK + NPV) {
        const int dt = (slot - NQK) / RT, rt = (slot - NQK) % RT;
        tw_mma16(acc[rt][dt], vf[dt], pb[rt]);
      } else {
        const int rt = slot - NQK - NPV;
        tw_mma16(l_mma[rt], ones, pb[rt]);                   // every output row: the sum over the block's keys
      }
#pragma unroll
      for (int q = slot * MPS; q < (slot + 1) * MPS; ++q) {
        if (q < NMEM) memory_operation(q);
        // The iteration's barrier stands in the middle of it: before it this wave's writes of block
        // blk + 2 and its last reads of block blk (whose stage the next iteration overwrites), behind it
        // the first reads of block blk + 2, which are in registers when the next iteration begins. A
        // wave in another kind of iteration has its barrier at the end, after the same writes and reads.
        if (q == VF_FIRST + DTMAX + NP - 1) __syncthreads();
      }
#pragma unroll
      for (int j = P_AHEAD; j < NPROB; ++j)
        if ((j - P_AHEAD) * P_SPAN / (NPROB - P_AHEAD) == slot) exponential(j);
#pragma unroll
      for (int k = 0; k < NMX; ++k)
        if (NQK + 2 + k * (NPV - 2) / NMX == slot) maximum(k);
      __builtin_amdgcn_sched_barrier(0);
    }
    move_reference(mx);
  };
  auto seen = [&](int blk) { return wave_live && blk < blk_end && blk * 32 <= wave_t_max; };
  auto edge_of = [&](int blk) {
    const int p0 = blk * 32;
    return !(p0 + 31 <= wave_t_min && p0 >= wave_lo_max && p0 + 32 <= kv_len);
  };
  // One iteration: block blk lies in stage buf and its scores in s_now; block blk + 1 lies in the next
  // stage, its scores go to s_then; block blk + 2, in registers since the iteration before, is written to
  // the stage after that (which held block blk - 1: every wave has left the iteration that read it), and
  // block blk + 3 is fetched. Fetches are unconditional (no register copies): past the end the last block
  // is fetched again.
  // The iterations in which the wave needs both steps and no masking (nearly all of them) run in a loop
  // of their own, whose body is one stretch of code without a branch between the two steps; what comes
  // before and after runs in loops whose body decides step by step. (One loop with both bodies behind a
  // branch made the compiler copy all 64 accumulators where the branches met.)
  f32x4 s_now[RT][2], s_then[RT][2];
  int blk = blk_begin, buf = 0;
  auto run_to = [&](int end, auto body) {
    for (; blk < end; ++blk) {
      const int buf1 = buf == TW_PF_STAGES - 1 ? 0 : buf + 1, buf2 = buf1 == TW_PF_STAGES - 1 ? 0 : buf1 + 1;
      body(blk, buf, buf1);
      // block blk + 2, fetched an iteration ago, goes to LDS; the registers it leaves take block blk + 3.
      // All of this stands behind the last MFMAs of the body, whose time it shares.
      stash(buf2);
      fetch(min(blk + 3, blk_end - 1));
      lookup(blk + 4);                                       // (its page numbers replace those just used)
      __syncthreads();
      buf = buf1;
      if constexpr (PIPELINED) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int tile = 0; tile < 2; ++tile) s_now[rt][tile] = s_then[rt][tile];
      }
    }
  };
  auto step_by_step = [&](int blk, int buf, int buf1) {
    if constexpr (PIPELINED) {
      // (the reference may move for block blk + 1 before block blk is added: the exponentials of both are
      // taken against the one that holds when they are formed, as sum and output are)
      if (seen(blk + 1)) {
        scores(blk + 1, buf1, edge_of(blk + 1), s_then);
        reference(s_then);
      }
      if (seen(blk)) finish(buf, s_now);
    } else if (seen(blk)) {
      scores(blk, buf, edge_of(blk), s_now);
      reference(s_now);
      finish(buf, s_now);
    }
  };
  auto both_steps = [&](int blk, int buf, int buf1) {
    finish_and_score(buf, buf1, s_now, s_then);
  };
  // both_steps for the blocks b of [both_begin, both_end): b + 1 is a block of this workgroup every key
  // of which every row of the wave sees (then so is b seen)
  int both_begin = blk_begin, both_end = blk_begin;
  if (PIPELINED && wave_live) {
    const int last_next = min(min(blk_end - 1, (wave_t_min + 1) / 32 - 1), kv_len / 32 - 1);   // the largest b + 1
    both_begin = max(blk_begin, (wave_lo_max + 31) / 32 - 1);
    both_end = max(both_begin, last_next);
  }

  lookup(blk_begin);
  fetch(blk_begin);
  lookup(blk_begin + 1);
  stash(0);
  fetch(min(blk_begin + 1, blk_end - 1));
  lookup(blk_begin + 2);
  stash(1);
  fetch(min(blk_begin + 2, blk_end - 1));
  lookup(blk_begin + 3);
  __syncthreads();
  if (PIPELINED && seen(blk_begin)) {
    scores(blk_begin, 0, edge_of(blk_begin), s_now);
    reference(s_now);
  }
  run_to(both_begin, step_by_step);
  if constexpr (EXACT && PIPELINED) {
    // (blk_end - 1 is the only block of the workgroup that may cross the end of the sequence)
    const bool all_whole = blk_end * 32 <= kv_len;
    const int ordered_end = all_whole ? both_end : min(both_end, blk_end - 5);
    bf16x8 ahead[KF_AHEAD];                                  // the first K fragments of the block after blk
    if (blk < ordered_end) {
      const int buf1 = buf == TW_PF_STAGES - 1 ? 0 : buf + 1;
#pragma unroll
      for (int k = 0; k < KF_AHEAD; ++k)
        ahead[k] = *reinterpret_cast<const bf16x8*>(k_frag[0] + buf1 * KSTAGE + (k & 1) * 16 * KROW + (k >> 1) * 64);
    }
    for (; blk < ordered_end; ++blk) {
      const int buf1 = buf == TW_PF_STAGES - 1 ? 0 : buf + 1, buf2 = buf1 == TW_PF_STAGES - 1 ? 0 : buf1 + 1;
      ordered_iteration(blk, buf, buf1, buf2, s_now, s_then, ahead);
      buf = buf1;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int tile = 0; tile < 2; ++tile) s_now[rt][tile] = s_then[rt][tile];
    }
  }
  run_to(both_end, both_steps);
  run_to(blk_end, step_by_step);                             // (blk_end > blk_begin always)
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) l[rt] = tw_rows_sum(l[rt]) + l_mma[rt][0];   // (the running maximum, and so every rescaling, was the row's: the same for the four)

  if (n_chunks > 1) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if (!row_ok[rt]) continue;
      const size_t slot = ((size_t)(token0 + tok[rt]) * a.q_heads + head[rt]) * a.max_chunks + chunk;
      float* dst = a.part_o + slot * D;
#pragma unroll
      for (int dt = 0; dt < DTMAX; ++dt)
        if (EXACT || dt < dts)
#pragma unroll
          for (int j = 0; j < 4; ++j) dst[dt * 16 + 4 * g + j] = acc[rt][dt][j];
      if (g == 0) {
        a.part_ml[slot * 2] = m[rt];                              // in the scaled log2 domain
        a.part_ml[slot * 2 + 1] = l[rt];
      }
    }
    return;
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (!row_ok[rt]) continue;
    const float inv = l[rt] > 0.f ? 1.f / l[rt] : 0.f;
    bf16_t* dst = (bf16_t*)a.out + (size_t)(token0 + tok[rt]) * a.ldo + (size_t)head[rt] * D;
#pragma unroll
    for (int dt = 0; dt < DTMAX; ++dt)
      if (EXACT || dt < dts)
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[dt * 16 + 4 * g + j] = (bf16_t)(acc[rt][dt][j] * inv);
  }
}

// Merge of the chunks of split tiles: grid = (8-row slices of the longest sequence's rows, kv_heads,
// n_seqs); a thread takes 4 output dims of one row, with the prefill kernel's own arithmetic for
// the key blocks of the row's tile. Chunks are added in index order.
#define TW_MERGE_ROWS 8          /* rows per workgroup: 32 threads each */
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(AttnArgs a) {
  const int G = a.q_heads / a.kv_heads;
  const int kvh = blockIdx.y, seq = a.seq0 + blockIdx.z;
  const int kv_len = a.kv_len[seq];
  const int token0 = a.q_start[seq];
  const int q_len = a.q_start[seq + 1] - token0;
  const int rows = q_len * G;
  const int D = a.head_dim, groups = D / 4;                      // groups of 4 output dims per row
  const int item = threadIdx.x;                                  // 32 threads per row
  const int row = blockIdx.x * TW_MERGE_ROWS + (item >> 5);
  if (row >= rows) return;
  const int wg_row0 = row / a.tile_rows * a.tile_rows;
  const int first_pos = kv_len - q_len;
  const int t_min = first_pos + wg_row0 / G;
  const int t_max = first_pos + min(rows - 1, wg_row0 + a.tile_rows - 1) / G;
  const int lo = a.window > 0 ? max(0, t_min - a.window + 1) : 0;
  const int tile_begin = lo / 32, tile_end = t_max / 32 + 1;
  const int chunk_blocks = a.kv_chunk / 32;
  const int n_chunks = (tile_end - tile_begin + chunk_blocks - 1) / chunk_blocks;
  if (n_chunks <= 1) return;                                     // the prefill kernel wrote the result itself
  const int tok = row / G, head = kvh * G + row % G;
  const size_t slot0 = ((size_t)(token0 + tok) * a.q_heads + head) * a.max_chunks;
  float m_all = -INFINITY;
  for (int c = 0; c < n_chunks; ++c) m_all = fmaxf(m_all, a.part_ml[(slot0 + c) * 2]);
  const float m_use = m_all == -INFINITY ? 0.f : m_all;
  for (int grp = item & 31; grp < groups; grp += 32) {
    float l_all = 0.f;
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int c = 0; c < n_chunks; ++c) {
      const float w = __builtin_amdgcn_exp2f(a.part_ml[(slot0 + c) * 2] - m_use);
      l_all += a.part_ml[(slot0 + c) * 2 + 1] * w;
      const f32x4 x = *reinterpret_cast<const f32x4*>(a.part_o + (slot0 + c) * D + grp * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] += x[e] * w;
    }
    const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
    bf16_t packed[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = (bf16_t)(o[e] * inv);
    bf16_t* dst = (bf16_t*)a.out + (size_t)(token0 + tok) * a.ldo + (size_t)head * D + grp * 4;
    *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(packed);
  }
}

// Rows of a workgroup's tile in the bfloat16 prefill kernel: 128 (32 per wave: half the LDS reads and a
// fifth fewer instructions a row), or 64 (16 per wave) where 128 would leave the chip with too few workgroups.
static int prefill_tile_rows(int n_seqs, int q_heads, int kv_heads, int max_q_len, int max_kv_len, int asked) {
  if (asked == 64 || asked == 128) return asked;
  const int G = kv_heads > 0 ? q_heads / kv_heads : 1;
  const long tiles128 = (long)tw_div_up((long)max_q_len * G, 128) * kv_heads * n_seqs;
  const long tiles64 = (long)tw_div_up((long)max_q_len * G, 64) * kv_heads * n_seqs;
  // Measured (28 query heads over 4, head size 128; us with 64-row / 128-row tiles).
  // A workgroup a CU or more without cutting tiles into chunks: 128. Whole prompts of 1,536 / 2,048 / 3,072 /
  // 4,096 tokens 42 / 40, 56 / 54, 110 / 88, 170 / 140; four of 512 25 / 22; 2,048 behind 1,024 cached 105 / 72.
  if (tiles128 >= 256) return 128;
  // A portion late in a long prompt (most keys come from the cache): every tile reads about max_kv_len
  // keys and what a row costs decides, also where the tiles are then cut into chunks: 256 / 512 / 1,024
  // tokens behind 8,192 cached 73 / 55, 122 / 98, 206 / 188.
  if (max_kv_len >= 2L * max_q_len && max_q_len >= 256 && max_kv_len >= 8192) return 128;
  // 64-row tiles fill the chip and 128-row tiles would have to be cut: 1,024 tokens alone 26 / 45, behind
  // 1,024 or 2,048 cached 42 / 66 and 66 / 85.
  if (tiles64 >= 256) return 64;
  // Both are cut into chunks: with few keys the shorter tiles (128 to 512 tokens alone: 19 / 21, 18 / 19,
  // 19 / 20), with many the cheaper rows (256 behind 2,048: 41 / 36; 128 behind 8,192: 41 / 38).
  return max_kv_len >= 2048 ? 128 : 64;
}

// How the keys of a prefill tile are split over workgroups: returns the most chunks a tile can
// have (1: no splitting) and the keys per chunk. With fewer tiles than the chip has room for,
// long tiles are cut so that there are about a thousand units of work of similar size.
// tile_rows: 0 (choose), 64 or 128; *tile_rows_out is the choice, to be given to tw_attn_prefill.
extern "C" int tw_attn_prefill_split(int n_seqs, int q_heads, int kv_heads, int max_q_len, int max_kv_len,
                                     int tile_rows_in, int* kv_chunk, int* tile_rows_out) {
  const int split_below = 256;                     // one tile per CU or more: tiles are left whole (measured)
  const int G = kv_heads > 0 ? q_heads / kv_heads : 1;
  const int tile_rows = prefill_tile_rows(n_seqs, q_heads, kv_heads, max_q_len, max_kv_len, tile_rows_in);
  *tile_rows_out = tile_rows;
  const long tiles = (long)tw_div_up((long)max_q_len * G, tile_rows) * kv_heads * n_seqs;
  *kv_chunk = 0;
  if (tiles <= 0 || tiles >= split_below || max_kv_len <= 512) return 1;
  int want = (int)tw_div_up(1024, tiles);
  if (want > 8) want = 8;
  int chunk = (int)tw_div_up(tw_div_up(max_kv_len, want), 32) * 32;
  if (chunk < 256) chunk = 256;
  const int chunks = (int)tw_div_up(max_kv_len + 31, chunk) + 1;     // a tile's first block may start mid-chunk
  if (chunks <= 1) return 1;
  *kv_chunk = chunk;
  return chunks;
}

extern "C" long tw_attn_prefill_workspace_floats(int n_tokens, int q_heads, int head_dim, int max_chunks) {
  return max_chunks > 1 ? (long)n_tokens * q_heads * max_chunks * (head_dim + 2) : 0;
}

template <int DTMAX, bool EXACT>
static int prefill_bf16_launch(AttnArgs a, int n_seqs, int max_q_len, hipStream_t stream) {
  const int G = a.q_heads / a.kv_heads;
  const long rows = (long)max_q_len * G;
  a.n_seqs = n_seqs;
  a.tile_rows = prefill_tile_rows(n_seqs, a.q_heads, a.kv_heads, max_q_len, 0, a.tile_rows);
  a.max_tiles = (int)tw_div_up(rows, a.tile_rows);
  const long total = (long)a.max_tiles * a.kv_heads * n_seqs * a.max_chunks;
  TW_REQUIRE(total < (1L << 30));
  TW_REQUIRE((long)a.kv_heads * a.page_size * a.head_dim * 2 < (1L << 31));      // a page's bytes: 32-bit in the kernel
  dim3 grid((unsigned)total);
  const size_t lds_bytes = TW_PF_STAGES * (32 * (DTMAX * 32 + 32) + DTMAX * 16 * TW_PF_VROW);
  static bool attribute_set = false;
  if (!attribute_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_bf16_kernel<DTMAX, EXACT, 1>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)attn_prefill_bf16_kernel<DTMAX, EXACT, 2>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return (int)e;
    attribute_set = true;
  }
  if (a.tile_rows == 64)
    attn_prefill_bf16_kernel<DTMAX, EXACT, 1><<<grid, 256, lds_bytes, stream>>>(a);
  else
    attn_prefill_bf16_kernel<DTMAX, EXACT, 2><<<grid, 256, lds_bytes, stream>>>(a);
  int err = TW_LAUNCH_RESULT();
  if (err || a.max_chunks <= 1) return err;
  attn_prefill_merge_kernel<<<dim3((unsigned)tw_div_up(rows, TW_MERGE_ROWS), a.kv_heads, n_seqs), 256, 0, stream>>>(a);
  return TW_LAUNCH_RESULT();
}

// =====================================================================================
// Host side
// =====================================================================================
static int check_common(const AttnArgs& a) {
  TW_REQUIRE(a.q_heads > 0 && a.kv_heads > 0 && a.q_heads % a.kv_heads == 0);
  TW_REQUIRE(a.head_dim >= 16 && a.head_dim <= 256 && a.head_dim % 16 == 0);
  TW_REQUIRE(a.page_size >= 4 && a.page_size % 4 == 0);
  TW_REQUIRE(a.window >= 0 && a.table_stride > 0);
  TW_REQUIRE(a.ldq >= (long)a.q_heads * a.head_dim && a.ldo >= (long)a.q_heads * a.head_dim);
  TW_REQUIRE(a.ldq % 8 == 0 && ((uintptr_t)a.q % 16 == 0));
  return 0;
}

// Key ranges per (sequence, kv head) of the decode kernel. One workgroup per CU is enough to stream (a
// wave keeps two 16 KB blocks in flight), and the kernel's time is that of the fullest CU: with `units`
// (sequence, kv head) pairs and s ranges each, ceil(units * s / 256) rounds of 1 / s of a pair's keys.
// The s with the least of that is taken, a percent per range added for the merge (288 workgroups, a
// few more than CUs, would take twice as long as 240).
extern "C" int tw_attn_decode_splits(int n_seqs, int q_heads, int kv_heads, int max_kv_len) {
  const int G = q_heads / kv_heads;
  const long units = (long)n_seqs * kv_heads * ((G + 15) / 16);
  int most = tw_div_up(max_kv_len, 256);                   // at least 256 keys a range
  if (most > 64) most = 64;
  int best = 1;
  double best_cost = 0;
  for (int s = 1; s <= most; ++s) {
    const double cost = (double)tw_div_up(units * s, 256) / s * (1.0 + 0.01 * s);
    if (s == 1 || cost < best_cost) {
      best = s;
      best_cost = cost;
    }
  }
  return best;
}

extern "C" long tw_attn_decode_workspace_floats(int n_seqs, int q_heads, int head_dim, int splits) {
  return splits > 1 ? (long)n_seqs * q_heads * splits * (head_dim + 2) : 0;
}

template <typename T> struct IsBf16 { static constexpr bool value = false; };
template <> struct IsBf16<bf16_t> { static constexpr bool value = true; };

template <typename T>
static int decode_launch(AttnArgs a, int n_seqs, int generic, hipStream_t stream) {
  const int G = a.q_heads / a.kv_heads;
  dim3 grid(a.splits, a.kv_heads * ((G + 15) / 16), n_seqs);
  if (IsBf16<T>::value && a.page_shift >= 3 && !generic) {
    if (a.head_dim == 64)
      attn_decode_bf16_kernel<4, true><<<grid, 256, 0, stream>>>(a);
    else if (a.head_dim < 64)
      attn_decode_bf16_kernel<4, false><<<grid, 256, 0, stream>>>(a);
    else if (a.head_dim == 128)
      attn_decode_bf16_kernel<8, true><<<grid, 256, 0, stream>>>(a);
    else if (a.head_dim < 128)
      attn_decode_bf16_kernel<8, false><<<grid, 256, 0, stream>>>(a);
    else if (a.head_dim == 256)
      attn_decode_bf16_kernel<16, true><<<grid, 256, 0, stream>>>(a);
    else
      attn_decode_bf16_kernel<16, false><<<grid, 256, 0, stream>>>(a);
  } else if (a.head_dim <= 64)
    attn_decode_kernel<T, 4><<<grid, 256, 0, stream>>>(a);
  else if (a.head_dim <= 128)
    attn_decode_kernel<T, 8><<<grid, 256, 0, stream>>>(a);
  else
    attn_decode_kernel<T, 16><<<grid, 256, 0, stream>>>(a);
  int err = TW_LAUNCH_RESULT();
  if (err || a.splits == 1) return err;
  attn_decode_reduce_kernel<T><<<dim3(a.q_heads, n_seqs), TW_REDUCE_THREADS, 0, stream>>>(
      a.part_o, a.part_ml, a.q_start, a.seq0, (T*)a.out, a.ldo, a.q_heads, a.head_dim, a.splits);
  return TW_LAUNCH_RESULT();
}

// Sequences seq0 .. seq0 + n_seqs - 1 must each have exactly one token in this step.
// `workspace` holds tw_attn_decode_workspace_floats floats when splits > 1.
// generic != 0 forces the kernel that takes every type and page size.
extern "C" int tw_attn_decode(int dtype, const void* q, long ldq, const void* keys, const void* values,
                              const int* block_table, int table_stride, const int* q_start,
                              const int* kv_len, int seq0, int n_seqs, void* out, long ldo,
                              float* workspace, long workspace_floats, int q_heads, int kv_heads,
                              int head_dim, int page_size, int window, float scale, float softcap, int splits,
                              int generic, hipStream_t stream) {
  AttnArgs a;
  a.q = q; a.ldq = ldq; a.keys = keys; a.values = values; a.block_table = block_table;
  a.table_stride = table_stride; a.q_start = q_start; a.kv_len = kv_len; a.seq0 = seq0;
  a.out = out; a.ldo = ldo; a.q_heads = q_heads; a.kv_heads = kv_heads; a.head_dim = head_dim;
  a.page_size = page_size; a.window = window; a.scale = scale; a.splits = splits;
  TW_REQUIRE(softcap >= 0.f);
  a.softcap = softcap;
  if (softcap > 0.f) generic = 1;
  a.part_o = nullptr; a.part_ml = nullptr;
  a.page_shift = -1;
  for (int sh = 0; sh < 20; ++sh)
    if ((1 << sh) == page_size) a.page_shift = sh;
  int err = check_common(a);
  if (err) return err;
  TW_REQUIRE(n_seqs >= 0 && seq0 >= 0 && splits >= 1 && splits <= 64 && n_seqs <= 65535);
  if (n_seqs == 0) return 0;
  if (splits > 1) {
    TW_REQUIRE(workspace != nullptr);
    TW_REQUIRE(workspace_floats >= tw_attn_decode_workspace_floats(n_seqs, q_heads, head_dim, splits));
    a.part_o = workspace;
    a.part_ml = workspace + (size_t)n_seqs * q_heads * splits * head_dim;
  }
  if (dtype == TW_DTYPE_F32) return decode_launch<float>(a, n_seqs, generic, stream);
  if (dtype == TW_DTYPE_BF16) return decode_launch<bf16_t>(a, n_seqs, generic, stream);
  return TW_ERR_BAD_ARGUMENT;
}

template <typename T>
static int prefill_launch(AttnArgs a, int n_seqs, int max_q_len, int generic, hipStream_t stream) {
  if (IsBf16<T>::value && a.page_shift >= 3 && !generic) {
    if (a.head_dim == 64) return prefill_bf16_launch<4, true>(a, n_seqs, max_q_len, stream);
    if (a.head_dim < 64) return prefill_bf16_launch<4, false>(a, n_seqs, max_q_len, stream);
    if (a.head_dim == 128) return prefill_bf16_launch<8, true>(a, n_seqs, max_q_len, stream);
    if (a.head_dim < 128) return prefill_bf16_launch<8, false>(a, n_seqs, max_q_len, stream);
    if (a.head_dim == 256) return prefill_bf16_launch<16, true>(a, n_seqs, max_q_len, stream);
    return prefill_bf16_launch<16, false>(a, n_seqs, max_q_len, stream);
  }
  const int G = a.q_heads / a.kv_heads;
  const long rows = (long)max_q_len * G;
  dim3 grid(tw_div_up(rows, 64), a.kv_heads, n_seqs);
  if (a.head_dim <= 64)
    attn_prefill_kernel<T, 4><<<grid, 256, 0, stream>>>(a);
  else if (a.head_dim <= 128)
    attn_prefill_kernel<T, 8><<<grid, 256, 0, stream>>>(a);
  else
    attn_prefill_kernel<T, 16><<<grid, 256, 0, stream>>>(a);
  return TW_LAUNCH_RESULT();
}

// Sequences seq0 .. seq0 + n_seqs - 1 with any number of tokens (at most max_q_len) each.
extern "C" int tw_attn_prefill(int dtype, const void* q, long ldq, const void* keys, const void* values,
                               const int* block_table, int table_stride, const int* q_start,
                               const int* kv_len, int seq0, int n_seqs, int max_q_len, void* out,
                               long ldo, float* workspace, long workspace_floats, int n_tokens, int max_chunks,
                               int kv_chunk, int tile_rows, int q_heads, int kv_heads, int head_dim, int page_size,
                               int window, float scale, float softcap, int generic, hipStream_t stream) {
  AttnArgs a;
  TW_REQUIRE(tile_rows == 0 || tile_rows == 64 || tile_rows == 128);
  a.tile_rows = tile_rows;
  a.q = q; a.ldq = ldq; a.keys = keys; a.values = values; a.block_table = block_table;
  a.table_stride = table_stride; a.q_start = q_start; a.kv_len = kv_len; a.seq0 = seq0;
  a.out = out; a.ldo = ldo; a.q_heads = q_heads; a.kv_heads = kv_heads; a.head_dim = head_dim;
  a.page_size = page_size; a.window = window; a.scale = scale; a.splits = 1;
  TW_REQUIRE(softcap >= 0.f);
  a.softcap = softcap;
  if (softcap > 0.f) generic = 1;
  a.part_o = nullptr; a.part_ml = nullptr;
  a.max_chunks = 1; a.kv_chunk = 0;
  a.page_shift = -1;
  for (int sh = 0; sh < 20; ++sh)
    if ((1 << sh) == page_size) a.page_shift = sh;
  int err = check_common(a);
  if (err) return err;
  TW_REQUIRE(n_seqs >= 0 && seq0 >= 0 && max_q_len >= 1 && n_seqs <= 65535);
  if (n_seqs == 0) return 0;
  // Splitting the keys of a tile (bfloat16 kernel only): partial results of token row n, head h, chunk c
  // at workspace[((n * q_heads + h) * max_chunks + c) * head_dim], their (maximum, sum) pairs behind them.
  if (max_chunks > 1 && workspace != nullptr) {
    TW_REQUIRE(kv_chunk >= 32 && kv_chunk % 32 == 0 && n_tokens >= 1);
    TW_REQUIRE(workspace_floats >= tw_attn_prefill_workspace_floats(n_tokens, q_heads, head_dim, max_chunks));
    TW_REQUIRE((uintptr_t)workspace % 16 == 0 && (uintptr_t)out % 16 == 0 && ldo % 8 == 0);
    a.max_chunks = max_chunks; a.kv_chunk = kv_chunk;
    a.part_o = workspace;
    a.part_ml = workspace + (size_t)n_tokens * q_heads * max_chunks * head_dim;
  }
  if (dtype == TW_DTYPE_F32) return prefill_launch<float>(a, n_seqs, max_q_len, generic, stream);
  if (dtype == TW_DTYPE_BF16) return prefill_launch<bf16_t>(a, n_seqs, max_q_len, generic, stream);
  return TW_ERR_BAD_ARGUMENT;
}
