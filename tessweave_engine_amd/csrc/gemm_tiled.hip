// Linear layers for many rows (prompt portions): LDS-staged MFMA tiles. See gemm.hip for the
// weight layouts and the GLU form; this file holds the kernel, its epilogue and its launcher.
#include "gemm_shared.h"

// Epilogue of the tiled kernels: each wave passes its tile through LDS (32 rows at a time) so
// that a lane stores 8 consecutive columns of one row, whole cache lines instead of 2- or 4-byte
// pieces; bias, residual, the output type and the SiLU-multiply of GLU pairs are applied here.
// `lds` must hold 4 waves x 32 rows x (32 * WN + 4) floats and no wave may still read its old contents
// (the first __syncthreads below sees to that).
template <typename OutT, int WM, int WN, bool GLU>
__device__ __forceinline__ void tw_tiled_epilogue(f32x16 (&acc)[WM][WN], char* lds, const float* __restrict__ bias,
                                                  const float* residual, long ldr, OutT* C, long ldc, int M, int N,
                                                  int m0, int n0, int wm0, int wn0, int wave, int lane) {
  const int r = lane & 31, g = lane >> 5;
  constexpr int WCOLS = 32 * WN;                             // columns of a wave tile
  constexpr int EROW = WCOLS + 4;                            // floats per staged row, padded
  // (the launcher asks for max(pipeline stages, 4 waves x 32 rows x EROW floats) bytes of LDS)
  float* stage = reinterpret_cast<float*>(lds) + wave * 32 * EROW;   // (the GLU form below may lay its rows out differently)
  constexpr int CPR = WCOLS / 8;                             // 8-column groups per row
  const bool vec_ok = (ldc % 8 == 0) && (residual == nullptr || ldr % 4 == 0) &&
                      ((uintptr_t)C % 16 == 0) && ((uintptr_t)residual % 16 == 0);
  // The GLU form reads its staged rows in another pattern: a lane takes 8 gate and 8 up values, 16 columns
  // apart, and the lanes of a row take column groups that are 256 bytes (all 64 banks) apart. With padded
  // rows those reads met 4-way bank conflicts (a quarter of the LDS time of a whole gate_up GEMM). Where a
  // wave tile's row is a multiple of 256 bytes the rows are not padded and the 16-byte pieces of row lr lie
  // at piece ^ (0, 1, 4, 5)[lr % 4]: the 16 lanes that a 16-byte read serves in one pass (four rows, four
  // column groups each) then find 16 different 16-byte columns.
  // Bias: a lane's group of 8 columns in its round t of a pass through LDS is group (lane + 64 t) % CPR of
  // the row, which repeats after NB rounds (1 where 64 is a multiple of the groups per row, 3 for 12 groups).
  // Those NB groups' bias is read once, before the first barrier, instead of eight values at a time in front of
  // every store (a fifth of a qkv projection's time at 2,048 rows went there).
  constexpr int NB = 64 % CPR == 0 ? 1 : ((128 % CPR == 0) ? 2 : 3);
  static_assert((64 * NB) % CPR == 0, "the column groups of a lane repeat after NB rounds");
  float lane_bias[NB][8];
  if (!GLU && bias) {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int col = n0 + wn0 + ((lane + 64 * b) % CPR) * 8;
      if (col + 8 <= N && (uintptr_t)bias % 16 == 0) {
        const f32x4 b0 = *reinterpret_cast<const f32x4*>(bias + col), b1 = *reinterpret_cast<const f32x4*>(bias + col + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { lane_bias[b][e] = b0[e]; lane_bias[b][4 + e] = b1[e]; }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) lane_bias[b][e] = col + e < N ? bias[col + e] : 0.f;
      }
    }
  }
  constexpr bool SWIZZLED = GLU && WCOLS % 64 == 0;
  constexpr int SROW = SWIZZLED ? WCOLS : EROW;
  if (SWIZZLED) stage = reinterpret_cast<float*>(lds) + wave * 32 * SROW;
  auto swz = [](int row) { return SWIZZLED ? ((row & 1) | ((row & 2) << 1)) : 0; };
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    __syncthreads();                                          // the pipeline's (or the last round's) LDS reads are done
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int srow = 8 * (e / 4) + 4 * g + (e % 4);
        stage[srow * SROW + (((j * 8 + (r >> 2)) ^ swz(srow)) << 2) + (r & 3)] = acc[i][j][e];
      }
    __syncthreads();
    if (GLU) {
      // a wave tile's columns are [gate 16 | up 16] pairs; a lane forms 8 outputs of one row
      constexpr int GPR = WCOLS / 16;                         // 8-output groups per row
#pragma unroll
      for (int q = lane; q < 32 * GPR; q += 64) {
        const int lr = q / GPR, og = q % GPR;
        const int lc = (og >> 1) * 32 + (og & 1) * 8;         // gate columns lc.., up columns lc + 16..
        const int row = m0 + wm0 + i * 32 + lr, col = n0 + wn0 + lc;
        if (row >= M || col + 24 > N) continue;               // N is a multiple of 32: groups are whole
        float v[8], gv[8], uv[8];
        if (SWIZZLED) {
          const float* base = stage + lr * SROW;
          const int piece = lc >> 2, x = swz(lr);
          const f32x4 g0 = *reinterpret_cast<const f32x4*>(base + ((piece ^ x) << 2));
          const f32x4 g1 = *reinterpret_cast<const f32x4*>(base + (((piece + 1) ^ x) << 2));
          const f32x4 u0 = *reinterpret_cast<const f32x4*>(base + (((piece + 4) ^ x) << 2));
          const f32x4 u1 = *reinterpret_cast<const f32x4*>(base + (((piece + 5) ^ x) << 2));
#pragma unroll
          for (int e = 0; e < 4; ++e) { gv[e] = g0[e]; gv[4 + e] = g1[e]; uv[e] = u0[e]; uv[4 + e] = u1[e]; }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) { gv[e] = stage[lr * SROW + lc + e]; uv[e] = stage[lr * SROW + lc + 16 + e]; }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if (bias) { gv[e] += bias[col + e]; uv[e] += bias[col + 16 + e]; }
          v[e] = tw_silu(gv[e]) * uv[e];
        }
        OutT* dst = C + (size_t)row * ldc + (n0 + wn0) / 2 + (og >> 1) * 16 + (og & 1) * 8;
        if (ldc % 8 == 0 && (uintptr_t)C % 16 == 0) {
          if (sizeof(OutT) == 4) {
            *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f32x4*>(dst + 4) = f32x4{v[4], v[5], v[6], v[7]};
          } else {
            bf16x8 o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (bf16_t)v[e];
            *reinterpret_cast<bf16x8*>(dst) = o;
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) dst[e] = tw_from_float<OutT>(v[e]);
        }
      }
      continue;
    }
#pragma unroll
    for (int t = 0; t < 32 * CPR / 64; ++t) {
      const int q = lane + 64 * t;
      const int lr = q / CPR, lc = (q % CPR) * 8;
      const int row = m0 + wm0 + i * 32 + lr, col = n0 + wn0 + lc;
      if (row >= M || col >= N) continue;
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = stage[lr * EROW + lc + e];
      if (bias) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += lane_bias[t % NB][e];
      }
      if (vec_ok && col + 8 <= N) {
        if (residual) {
          const f32x4 r0 = *reinterpret_cast<const f32x4*>(residual + (size_t)row * ldr + col);
          const f32x4 r1 = *reinterpret_cast<const f32x4*>(residual + (size_t)row * ldr + col + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) { v[e] += r0[e]; v[4 + e] += r1[e]; }
        }
        OutT* dst = C + (size_t)row * ldc + col;
        if (sizeof(OutT) == 4) {
          *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
          *reinterpret_cast<f32x4*>(dst + 4) = f32x4{v[4], v[5], v[6], v[7]};
        } else {
          bf16x8 o;
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = (bf16_t)v[e];
          *reinterpret_cast<bf16x8*>(dst) = o;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < N) {
            float x = v[e];
            if (residual) x += residual[(size_t)row * ldr + col + e];
            C[(size_t)row * ldc + col + e] = tw_from_float<OutT>(x);
          }
      }
    }
  }
}

// =====================================================================================
// Tiled kernel. Workgroup = 4 waves in a 2x2 grid, wave tile (32*WM) x (32*WN): tiles of 128x128
// (two workgroups per CU), 128x256 and 256x256 (one per CU, the accumulators in AGPRs).
// One stage holds 128 bytes of K per row (64 bf16 / 32 f32), rows padded to 144
// bytes in LDS so that 16-byte fragment reads of 8 consecutive lanes hit
// distinct banks. Two stages: the next stage's global loads are in flight
// while the current one is multiplied.
// =====================================================================================
#define TW_LDS_ROW 144

// SHUF: W is in the shuffled layout and ldw is its k_steps. GLU: see the top of the file.
template <typename T, typename OutT, int WM, int WN, bool SHUF, bool GLU>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const T* __restrict__ A, long lda,
                                                         const T* __restrict__ W, long ldw,
                                                         const float* __restrict__ bias,
                                                         const float* residual, long ldr, OutT* C,
                                                         long ldc, int M, int N, int K, int tiles_m,
                                                         int n_blocks, int splits, float* __restrict__ partial) {
  typedef typename Elem<T>::Frag Frag;
  constexpr int EPF = Elem<T>::kPerFrag;
  constexpr int KCH = 8;                                    // 16-byte chunks of K per row and stage
  constexpr int BK = KCH * EPF;
  constexpr int BM = 64 * WM, BN = 64 * WN;
  constexpr int LROW = KCH * 16 + 16;                       // LDS bytes per row of a stage, padded
  constexpr int A_LOADS = BM * KCH / 256, W_LOADS = BN * KCH / 256;
  constexpr int STAGE = (BM + BN) * LROW;                   // bytes of one stage: A rows then W rows
  extern __shared__ __attribute__((aligned(16))) char lds[];

  // Blocks are dealt to the 8 XCDs round-robin; give each XCD a contiguous run
  // of tiles so that neighbours sharing a weight tile share an L2.
  const int per_xcd = gridDim.x / 8;
  const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (logical >= n_blocks) return;
  // splits > 1 (few tiles, long K): the k-tiles are dealt to `splits` workgroups per tile, which
  // leave float32 partial sums partial[split][M][N] for splitk_reduce_kernel.
  const int n_tiles = n_blocks / splits;
  const int split = logical / n_tiles, tile = logical % n_tiles;
  // Tiles in bands of 2,048 rows, so that the workgroups an XCD runs at a time share column tiles as
  // well as row tiles (all the row tiles of a tall matrix in one column would share one weight tile
  // and fetch an activation tile each).
  constexpr int BAND = 2048 / BM;
  const int tiles_n = n_tiles / tiles_m;
  const int band = tile / (BAND * tiles_n), in_band = tile - band * BAND * tiles_n;
  const int band_rows = min(BAND, tiles_m - band * BAND);
  const int tile_m = band * BAND + in_band % band_rows, tile_n = in_band / band_rows;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 32 * WM, wn0 = (wave & 1) * 32 * WN;
  const int r = lane & 31, g = lane >> 5;

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // Global addressing: a tile base that is the same for every lane, plus per-thread element
  // offsets fixed for the whole K loop. Rows past the end are clamped to the last valid row
  // (what they produce is never stored), so whole k-tiles need no predicate.
  const T* a_tile = A + (size_t)m0 * lda;
  const T* w_tile = SHUF ? W + (size_t)(n0 / 16) * ldw * 64 * EPF : W + (size_t)n0 * ldw;
  const int k_steps_w = SHUF ? (int)ldw : 0;
  unsigned a_off[A_LOADS], w_off[W_LOADS];
  int st_off[A_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    const int c = tid + i * 256, row = c / KCH, kc = c % KCH;
    a_off[i] = (unsigned)(min(m0 + row, M - 1) - m0) * (unsigned)lda + kc * EPF;
  }
  constexpr int SPT = KCH / 4;                             // shuffled k-steps per k-tile
  int w_st_off[W_LOADS], w_ks[W_LOADS];
  const int n_blocks_w = (N + 15) / 16;
#pragma unroll
  for (int i = 0; i < W_LOADS; ++i) {
    const int c = tid + i * 256;
    if (SHUF) {
      // piece c of the tile: block (16 rows x 4 chunks) c / 64, lane c % 64 of that block
      const int blk = c >> 6, ln = c & 63, nblk = blk / SPT, ks = blk % SPT;
      const int gblk = min(n0 / 16 + nblk, n_blocks_w - 1);
      w_off[i] = (unsigned)(gblk - n0 / 16) * (unsigned)ldw * 64 * EPF + (ks * 64 + ln) * EPF;
      w_ks[i] = ks;
      w_st_off[i] = (nblk * 16 + (ln & 15)) * LROW + (ks * 4 + (ln >> 4)) * 16;
    } else {
      const int row = c / KCH, kc = c % KCH;
      w_off[i] = (unsigned)(min(n0 + row, N - 1) - n0) * (unsigned)ldw + kc * EPF;
      w_ks[i] = 0;
      w_st_off[i] = row * LROW + kc * 16;
    }
  }
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    const int c = tid + i * 256, row = c / KCH, kc = c % KCH;
    st_off[i] = row * LROW + kc * 16;
  }
  const int kc_mine = tid % KCH;

  // Two register sets: the global loads of k-tile kt+2 are issued while k-tile kt is multiplied,
  // so two k-tiles per workgroup are on their way from memory at any time.
  Frag a_regs[2][A_LOADS], w_regs[2][W_LOADS];
  const int k_tiles_all = (K + BK - 1) / BK;
  const int per_split = (k_tiles_all + splits - 1) / splits;
  const int kt0 = split * per_split;                          // this workgroup's k-tiles: kt0 .. kt0 + k_tiles - 1
  const int k_tiles = max(0, min(k_tiles_all, kt0 + per_split) - kt0);
  const int whole_tiles = K / BK;

  // whole k-tiles need no predicate at all; the main loop below runs only those
  auto load_whole = [&](int kt, Frag* a_reg, Frag* w_reg) {
    const T* ab = a_tile + (size_t)kt * BK;
    const T* wb = SHUF ? w_tile + (size_t)kt * SPT * 64 * EPF : w_tile + (size_t)kt * BK;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) a_reg[i] = tw_load_frag(ab + a_off[i]);
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) w_reg[i] = tw_load_frag(wb + w_off[i]);
  };
  auto load_global = [&](int kt, Frag* a_reg, Frag* w_reg) {
    if (kt < whole_tiles) {
      load_whole(kt, a_reg, w_reg);
    } else {                                                // the last, partial k-tile: chunks past K are zeros
      const T* ab = a_tile + (size_t)kt * BK;
      const T* wb = SHUF ? w_tile + (size_t)kt * SPT * 64 * EPF : w_tile + (size_t)kt * BK;
      const bool ok = kt * BK + kc_mine * EPF < K;
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) a_reg[i] = ok ? tw_load_frag(ab + a_off[i]) : Elem<T>::zero();
#pragma unroll
      for (int i = 0; i < W_LOADS; ++i) {
        const bool w_ok = SHUF ? kt * SPT + w_ks[i] < k_steps_w : ok;     // the shuffled layout is zero padded
        w_reg[i] = w_ok ? tw_load_frag(wb + w_off[i]) : Elem<T>::zero();
      }
    }
  };
  auto store_lds = [&](int buf, const Frag* a_reg, const Frag* w_reg) {
    char* base = lds + buf * STAGE;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) *reinterpret_cast<Frag*>(base + st_off[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) *reinterpret_cast<Frag*>(base + BM * LROW + w_st_off[i]) = w_reg[i];
  };

  // this lane's fragment addresses in stage 0 (k-chunk pair cc adds 32 bytes)
  const char* a_frag = lds + (wm0 + r) * LROW + g * 16;
  const char* w_frag = lds + (BM + wn0 + r) * LROW + g * 16;
  auto read_frags = [&](int buf, int cc, Frag* af, Frag* wf) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
      af[i] = *reinterpret_cast<const Frag*>(a_frag + buf * STAGE + i * 32 * LROW + cc * 32);
#pragma unroll
    for (int j = 0; j < WN; ++j)
      wf[j] = *reinterpret_cast<const Frag*>(w_frag + buf * STAGE + j * 32 * LROW + cc * 32);
  };

  auto multiply = [&](int buf) {
    // the fragments of the next k-chunk pair are read from LDS while this one is multiplied
    Frag af[2][WM], wf[2][WN];
    read_frags(buf, 0, af[0], wf[0]);
#pragma unroll
    for (int cc = 0; cc < KCH / 2; ++cc) {
      if (cc + 1 < KCH / 2) read_frags(buf, cc + 1, af[(cc + 1) & 1], wf[(cc + 1) & 1]);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) tw_mma32(acc[i][j], af[cc & 1][i], wf[cc & 1][j]);
    }
  };

  if (k_tiles > 0) {
    load_global(kt0, a_regs[0], w_regs[0]);
    if (k_tiles > 1) load_global(kt0 + 1, a_regs[1], w_regs[1]);
    store_lds(0, a_regs[0], w_regs[0]);
  }
  __syncthreads();
  int j = 0;                                                  // k-tile kt0 + j is in LDS stage j & 1
  // Main loop: two k-tiles per round, every load whole and unconditional, so that the register
  // sets are plain loop-carried values (conditional loads cost a register copy per loaded dword).
  const int whole_here = min(k_tiles, whole_tiles - kt0);
  // The order asked of the scheduler for each k-tile: per k-chunk pair its MFMAs, before them the
  // LDS reads of the next pair, a quarter of the next-but-one k-tile's global loads and a quarter of
  // the next k-tile's LDS writes. Left alone, the compiler puts loads, writes and MFMAs in three
  // clusters, and the memory pipes and the matrix unit take turns instead of working side by side.
#define TW_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define TW_TILE_ORDER()                                                                     \
  do {                                                                                      \
    constexpr int MOVES = (A_LOADS + W_LOADS) / 4;                                          \
    TW_SGB(0x100, WM + WN);                                                                 \
    TW_SGB(0x100, WM + WN); TW_SGB(0x020, MOVES); TW_SGB(0x200, MOVES); TW_SGB(0x008, WM * WN); \
    TW_SGB(0x100, WM + WN); TW_SGB(0x020, MOVES); TW_SGB(0x200, MOVES); TW_SGB(0x008, WM * WN); \
    TW_SGB(0x100, WM + WN); TW_SGB(0x020, MOVES); TW_SGB(0x200, MOVES); TW_SGB(0x008, WM * WN); \
    TW_SGB(0x020, MOVES); TW_SGB(0x200, MOVES); TW_SGB(0x008, WM * WN);                     \
  } while (0)
  for (; j + 3 < whole_here; j += 2) {
    load_whole(kt0 + j + 2, a_regs[0], w_regs[0]);           // LDS stage 0, register set 0 is free
    multiply(0);
    store_lds(1, a_regs[1], w_regs[1]);
    TW_TILE_ORDER();
    __syncthreads();
    load_whole(kt0 + j + 3, a_regs[1], w_regs[1]);           // LDS stage 1, register set 1 is free
    multiply(1);
    store_lds(0, a_regs[0], w_regs[0]);
    TW_TILE_ORDER();
    __syncthreads();
  }
#undef TW_TILE_ORDER
#undef TW_SGB
  // The last few k-tiles (j is even here): the same rounds with every step conditional.
  for (; j < k_tiles; j += 2) {
    if (j + 2 < k_tiles) load_global(kt0 + j + 2, a_regs[0], w_regs[0]);
    multiply(0);
    if (j + 1 < k_tiles) store_lds(1, a_regs[1], w_regs[1]);
    __syncthreads();
    if (j + 1 >= k_tiles) break;
    if (j + 3 < k_tiles) load_global(kt0 + j + 3, a_regs[1], w_regs[1]);
    multiply(1);
    if (j + 2 < k_tiles) store_lds(0, a_regs[0], w_regs[0]);
    __syncthreads();
  }

  if (splits > 1) {
    tw_tiled_epilogue<float, WM, WN, false>(acc, lds, nullptr, nullptr, 0, partial + (size_t)split * M * N, (long)N,
                                            M, N, m0, n0, wm0, wn0, wave, lane);
    return;
  }
  tw_tiled_epilogue<OutT, WM, WN, GLU>(acc, lds, bias, residual, ldr, C, ldc, M, N, m0, n0, wm0, wn0, wave, lane);
}

// =====================================================================================
// bfloat16, shuffled weights, K a multiple of 32: tiles whose operands are copied from global
// memory straight into LDS (`global_load_lds_dwordx4`: lane l's 16 bytes land at the wave's LDS
// base + 16 l, from any address the lane names). No staging registers, no LDS write instructions.
// Workgroup = 4 waves in a 2x2 grid, wave tile (32*WM) x (32*WN): 128x128 (two workgroups a CU),
// 128x256, 256x256 (one a CU, the accumulators in AGPRs).
//
// A k-tile is 32 elements of K (one k-step of the shuffled layout). What limits this kernel is the
// number of 128-byte lines a CU's vector cache can have on their way from L2; a copy that takes 64 bytes
// of a row of A brings in the whole line, and by the time the next k-tile wants the other half the line
// is gone again (measured: 1.5 lines fetched per line used). So A is copied in PAIRS of k-tiles, a
// whole line per row: a copy is 8 rows x 128 bytes, and LDS holds TW_DMA_A_SLOTS slots of BM rows x 128
// bytes. In a slot row `row` keeps its 16-byte chunk c (0..3: the even k-tile, 4..7: the odd one) at
// position c ^ (row / 2 % 8), so that the 16 rows one fragment read takes lie in 16 different 16-byte
// columns. W is copied per k-tile into 4 stages; a W block is 16 rows x 4 chunks, [chunk][row], 1 KB,
// which is how W lies in memory (a fragment read takes 256 consecutive bytes per 16 lanes).
//
// Per k-tile and wave: 2 k-chunk pairs of WM*WN MFMAs. The fragments of a pair are read while the
// pair before is multiplied, so the barrier that publishes the next k-tile lies between the two
// pairs of this one and the matrix unit has work queued on both sides of it.
// splits > 1: as in gemm_tiled_kernel (a split's k-tiles begin at an even one).
// =====================================================================================
typedef __attribute__((address_space(3))) void* tw_lds_ptr;
#define TW_DMA_STAGES 4       /* of W, one k-tile each */
#define TW_DMA_A_SLOTS 3      /* of A, a pair of k-tiles each */

// f(integral_constant<int, 0>), ..., f(integral_constant<int, N - 1>): a loop whose index is a constant
// expression in the body (the scheduler's group barriers take constants only)
template <int... Is, typename F>
__device__ __forceinline__ void tw_unroll_impl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void tw_unroll(F&& f) {
  tw_unroll_impl(std::make_integer_sequence<int, N>{}, f);
}

template <typename OutT, int WM, int WN, bool GLU>
__global__ __launch_bounds__(256) void gemm_dma_kernel(const bf16_t* __restrict__ A, long lda,
                                                       const bf16_t* __restrict__ W, long k_steps,
                                                       const float* __restrict__ bias, const float* residual,
                                                       long ldr, OutT* C, long ldc, int M, int N, int K,
                                                       int tiles_m, int n_blocks, int splits,
                                                       float* __restrict__ partial) {
  static_assert(WM % 2 == 0, "the tail fix below assumes an even number of A copies per group");
  constexpr int BM = 64 * WM, BN = 64 * WN;
  constexpr int A_SLOT = BM * 128;                      // bytes: a pair of k-tiles of A
  constexpr int W_STAGE = BN * 64;                      // bytes: one k-tile of W
  constexpr int W_RING = TW_DMA_A_SLOTS * A_SLOT;       // the W stages lie behind the A slots
  constexpr int COPIES = WM + WN;                       // 1 KB copies per wave and k-tile
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int per_xcd = gridDim.x / 8;
  const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;   // neighbours in an XCD share operand tiles
  if (logical >= n_blocks) return;
  const int n_tiles = n_blocks / splits;
  const int split = logical / n_tiles, tile = logical % n_tiles;
  // Tiles in bands of 2,048 rows: the workgroups an XCD runs at a time then share column tiles as well
  // as row tiles (all the row tiles of a tall matrix in one column would fetch an activation tile each).
  constexpr int BAND = 2048 / BM;
  const int tiles_n = n_tiles / tiles_m;
  const int band = tile / (BAND * tiles_n), in_band = tile - band * BAND * tiles_n;
  const int band_rows = min(BAND, tiles_m - band * BAND);
  const int tile_m = band * BAND + in_band % band_rows, tile_n = in_band / band_rows;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave >> 1) * 32 * WM, wn0 = (wave & 1) * 32 * WN;
  const int r = lane & 31, g = lane >> 5;

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // this workgroup's k-tiles: kt0 .. kt0 + k_tiles - 1, kt0 even (a pair of k-tiles is never divided)
  const int k_tiles_all = K / 32;
  const int per_split = ((k_tiles_all + splits - 1) / splits + 1) & ~1;
  const int kt0 = split * per_split;
  const int k_tiles = max(0, min(k_tiles_all, kt0 + per_split) - kt0);
  const int pairs = (k_tiles + 1) / 2;
  const bool half_pair = (k_tiles & 1) != 0;               // the last pair has its even k-tile only

  // What this lane copies: per pair of k-tiles its slot of the A blocks (8 rows each) 2 WM wave ..
  // 2 WM wave + 2 WM - 1, in two groups of WM, and per k-tile its slot of the W blocks (16 rows each)
  // WN wave .. WN wave + WN - 1. Rows past M and blocks past N are clamped to the last valid one (their
  // products are never stored).
  const int n_blocks_w = (N + 15) / 16;
  // (A: byte offsets from the tile's first row, for group 0 and from group 0 to group 1; which group a
  // copy belongs to is not known where it is compiled, and a choice between two pointers would put them
  // into memory)
  const char* const a_base = reinterpret_cast<const char*>(A + (size_t)m0 * lda + (size_t)kt0 * 32);
  int a_off[WM], a_step[WM];
  const bf16_t* w_src[WN];
#pragma unroll
  for (int b = 0; b < WM; ++b) {
    int off[2];
#pragma unroll
    for (int grp = 0; grp < 2; ++grp) {
      const int row_in_tile = ((2 * WM) * wave + grp * WM + b) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((row_in_tile >> 1) & 7);   // slot l % 8 of the row holds this chunk
      off[grp] = min(row_in_tile, M - 1 - m0) * (int)lda * 2 + chunk * 16;
    }
    a_off[b] = off[0];
    a_step[b] = off[1] - off[0];
  }
#pragma unroll
  for (int b = 0; b < WN; ++b) {
    const int blk = min(n0 / 16 + WN * wave + b, n_blocks_w - 1);
    w_src[b] = W + ((size_t)blk * k_steps + kt0) * 512 + lane * 8;
  }
  // In a last pair that has its even k-tile only, the lanes that would fetch chunks 4..7 (past the end of
  // the row, and for the last row perhaps of the matrix) fetch chunks 0..3 again. Whether a lane's chunk
  // is 4..7: bit 2 of l % 8, flipped in every other block of 8 rows.
  const int tail_back[2] = {(lane & 4) ? -64 : 0, (lane & 4) ? 0 : -64};   // bytes
  auto copy_a_one = [&](int pair_v, int grp, int b) {       // (grp, 0 or 1, is the same for the whole wave)
    const int pair = min(pair_v, pairs - 1);               // past the end: a copy nobody reads
    const int tail = (half_pair && pair == pairs - 1) ? -1 : 0;
    char* slot = lds + (pair_v % TW_DMA_A_SLOTS) * A_SLOT;
    const int off = a_off[b] + (a_step[b] & -grp) + (tail_back[b & 1] & tail);
    __builtin_amdgcn_global_load_lds((const void*)(a_base + (size_t)pair * 128 + (long)off),
                                     (tw_lds_ptr)(slot + ((2 * WM) * wave + grp * WM + b) * 1024), 16, 0, 0);
  };
  auto copy_w_one = [&](int t_v, int b) {
    const int t = min(t_v, k_tiles - 1);
    char* stage = lds + W_RING + (t_v % TW_DMA_STAGES) * W_STAGE;
    __builtin_amdgcn_global_load_lds((const void*)(w_src[b] + (size_t)t * 512), (tw_lds_ptr)(stage + (WN * wave + b) * 1024), 16, 0, 0);
  };
  // this lane's fragment offsets: A in slot 0 for the k-chunk pairs of an even k-tile (an odd one's
  // chunks are 4 further on: bit 6 of the offset flipped), W in stage 0
  const int a_swz = (r >> 1) & 7;
  const int a_frag[2] = {(wm0 + r) * 128 + ((g ^ a_swz) * 16), (wm0 + r) * 128 + (((2 + g) ^ a_swz) * 16)};
  const char* w_frag = lds + W_RING + (wn0 / 16 + (r >> 4)) * 1024 + g * 256 + (r & 15) * 16;
  // Wait until at most `count` of this wave's copies are in flight (copies finish in order), then meet the
  // other waves. The count is an immediate of the instruction, hence the cases.
#define TW_DMA_WAIT(n) asm volatile("s_waitcnt vmcnt(" #n ") lgkmcnt(0)" ::: "memory")
#define TW_DMA_PUBLISH(count)                                                 \
  do {                                                                        \
    if constexpr ((count) == 6) TW_DMA_WAIT(6);                               \
    else if constexpr ((count) == 8) TW_DMA_WAIT(8);                          \
    else if constexpr ((count) == 10) TW_DMA_WAIT(10);                        \
    else if constexpr ((count) == 12) TW_DMA_WAIT(12);                        \
    else if constexpr ((count) == 14) TW_DMA_WAIT(14);                        \
    else if constexpr ((count) == 16) TW_DMA_WAIT(16);                        \
    else TW_DMA_WAIT(0);                                                      \
    __builtin_amdgcn_s_barrier();                                             \
    asm volatile("" ::: "memory");                                            \
  } while (0)
#define TW_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)

  bf16x8 af[2][WM], wf[2][WN];
  // One wave a SIMD issues in order, and the matrix unit takes an MFMA every 32 clocks: whatever else
  // the wave issues between two MFMAs has to fit into that time, or the unit idles. So the other
  // operations of a k-chunk pair follow its MFMAs one by one: first the fragment reads of the next pair
  // (into the other set of registers), then the copies: the W blocks of k-tile t + 3 in the first pair of
  // k-tile t, one group of the A blocks of k-tile pair t / 2 + 2 in the second (the slot those land in
  // held pair t / 2 - 1, last read before the barrier of k-tile 2 (t / 2) - 1). The last MFMAs of a pair
  // have nothing behind them: a copy counts as an access through both memory counters, after which every
  // wait the compiler puts before an MFMA whose operands came from LDS is `lgkmcnt(0)`, and the one before
  // the next pair's first MFMA should find the reads long done. The source is written in the order that
  // is wanted, because a copy writes LDS and the compiler keeps LDS reads on their side of it; the group
  // barriers only pin it.
  auto half = [&](auto copy_is_a, int copy_index, int copy_group, const char* a_read, const char* w_read,
                  bf16x8* af_in, bf16x8* wf_in, bf16x8* af_out, bf16x8* wf_out) {
    constexpr bool IS_A = decltype(copy_is_a)::value;
    constexpr int NCOPY = IS_A ? WM : WN;
    // S slots of one MFMA each; the Q other operations (R fragment reads, then the copies) follow the
    // MFMAs of the first slots one by one (two where there are more operations than slots)
    constexpr int S = WM * WN, R = WM + WN, Q = R + NCOPY;
    tw_unroll<S>([&](auto index) {
      constexpr int slot = decltype(index)::value, i = slot / WN, j = slot % WN;
      tw_mma32(acc[i][j], af_in[i], wf_in[j]);
      constexpr int q0 = Q <= S ? (slot < Q ? slot : Q) : slot * Q / S;
      constexpr int q1 = Q <= S ? (slot + 1 < Q ? slot + 1 : Q) : (slot + 1) * Q / S;
#pragma unroll
      for (int q = q0; q < q1; ++q) {
        if (q < WM) af_out[q] = *reinterpret_cast<const bf16x8*>(a_read + q * 4096);
        else if (q < R) wf_out[q - WM] = *reinterpret_cast<const bf16x8*>(w_read + (q - WM) * 2048);
        else if (IS_A) copy_a_one(copy_index, copy_group, q - R);
        else copy_w_one(copy_index, q - R);
      }
      constexpr int reads_here = (q1 < R ? q1 : R) - (q0 < R ? q0 : R), copies_here = (q1 - q0) - reads_here;
      TW_SGB(0x008, 1);
      if constexpr (reads_here > 0) TW_SGB(0x100, reads_here);
      if constexpr (copies_here > 0) TW_SGB(0x020, copies_here);
    });
  };
  // k-tile t. Its barrier publishes k-tile t + 1. What has to have landed by then and what this wave
  // has issued since: t + 1 odd: W of t + 1 (issued in the first pair of t - 2), since then A, W A, W;
  // t + 1 even: its pair of A, whose second group went out in the second pair of t - 2, since then W A, W.
  // One count for both (the parity of t is not known where the wait is compiled): the smaller.
  auto k_tile = [&](int t) {
    const int odd = t & 1;
    const int a_now = ((t >> 1) % TW_DMA_A_SLOTS) * A_SLOT, a_next = (((t + 1) >> 1) % TW_DMA_A_SLOTS) * A_SLOT;
    const int w_now = (t % TW_DMA_STAGES) * W_STAGE, w_next = ((t + 1) % TW_DMA_STAGES) * W_STAGE;
    half(std::false_type{}, t + TW_DMA_STAGES - 1, 0, lds + ((a_frag[1] ^ (odd << 6)) + a_now), w_frag + w_now + 512,
         af[0], wf[0], af[1], wf[1]);
    __builtin_amdgcn_sched_barrier(0);                     // (nothing of either pair moves across the barrier)
    TW_DMA_PUBLISH(2 * WN + WM);
    __builtin_amdgcn_sched_barrier(0);
    half(std::true_type{}, (t >> 1) + 2, odd, lds + ((a_frag[0] ^ ((odd ^ 1) << 6)) + a_next), w_frag + w_next,
         af[1], wf[1], af[0], wf[0]);                      // (after the last k-tile: read, never used)
    __builtin_amdgcn_sched_barrier(0);                     // (nor into the next k-tile)
  };
  if (k_tiles > 0) {
    // A of pair 0 and W of k-tile 0, then what may still be on its way when k-tile 0 is published:
    // W of k-tile 1, A of pair 1, W of k-tile 2
#pragma unroll
    for (int c = 0; c < 2 * WM; ++c) copy_a_one(0, c / WM, c % WM);
#pragma unroll
    for (int b = 0; b < WN; ++b) copy_w_one(0, b);
#pragma unroll
    for (int b = 0; b < WN; ++b) copy_w_one(1, b);
#pragma unroll
    for (int c = 0; c < 2 * WM; ++c) copy_a_one(1, c / WM, c % WM);
#pragma unroll
    for (int b = 0; b < WN; ++b) copy_w_one(2, b);
    TW_DMA_PUBLISH(2 * COPIES);
#pragma unroll
    for (int i = 0; i < WM; ++i) af[0][i] = *reinterpret_cast<const bf16x8*>(lds + a_frag[0] + i * 4096);
#pragma unroll
    for (int j = 0; j < WN; ++j) wf[0][j] = *reinterpret_cast<const bf16x8*>(w_frag + j * 2048);
    for (int t = 0; t < k_tiles; ++t) k_tile(t);
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // no copy may land in the epilogue's staging area
#undef TW_SGB
#undef TW_DMA_PUBLISH
#undef TW_DMA_WAIT
  if (splits > 1) {
    tw_tiled_epilogue<float, WM, WN, false>(acc, lds, nullptr, nullptr, 0, partial + (size_t)split * M * N, (long)N,
                                            M, N, m0, n0, wm0, wn0, wave, lane);
    return;
  }
  tw_tiled_epilogue<OutT, WM, WN, GLU>(acc, lds, bias, residual, ldr, C, ldc, M, N, m0, n0, wm0, wn0, wave, lane);
}

// =====================================================================================
// Host side
// =====================================================================================
// How many K ranges the tiled kernel uses: with fewer tiles than the chip has room for (a prompt
// portion of a few hundred rows against a square or tall matrix) the k-tiles of a tile are dealt
// to several workgroups. Depends on the shape only.
// How a launch may deviate from "compute C": `leave` keeps the float32 sums of the K ranges in `partial`
// for the caller's next kernel (no reduction kernel; the caller passes C = partial as float32 without
// bias or residual, so that with a single range the product itself is partial[0]); `dry` launches
// nothing and only reports, in `splits`, the number of K ranges the launch would use.
struct TiledMode {
  bool leave = false, dry = false;
  int splits = 0;
};

static int tiled_splits(int M, int N, int K, int epf, int bm, int bn) {
  const long tiles = (long)tw_div_up(M, bm) * tw_div_up(N, bn);
  if (tiles >= 192) return 1;
  const int k_tiles = tw_div_up(K, 8 * epf);
  long splits = tw_div_up(384, tiles);
  const long resident = (long)bm * bn <= 128 * 128 ? 512 : 256;   // workgroups the chip holds at once
  if (splits > resident / tiles) splits = resident / tiles;       // never a few more than that: a second round
  if (splits > k_tiles / 8) splits = k_tiles / 8;
  if (splits > 8) splits = 8;
  return splits < 1 ? 1 : (int)splits;
}

template <typename T, typename OutT, int WM, int WN, bool SHUF, bool GLU>
static int launch_tiled(const T* A, long lda, const T* W, long ldw, const float* bias,
                        const float* residual, long ldr, OutT* C, long ldc, float* partial,
                        long partial_bytes, int M, int N, int K, int want_splits, hipStream_t stream,
                        TiledMode* mode = nullptr) {
  constexpr int BM = 64 * WM, BN = 64 * WN, KCH = 8;
  constexpr int EPF = Elem<T>::kPerFrag;
  const int tiles_m = tw_div_up(M, BM), tiles_n = tw_div_up(N, BN);
  int splits = GLU ? 1 : (want_splits > 0 ? want_splits : tiled_splits(M, N, K, EPF, BM, BN));
  if (mode && mode->dry) {
    mode->splits = splits;
    return 0;
  }
  if (splits > 1 && (partial == nullptr || partial_bytes < (long)splits * M * N * 4 || (uintptr_t)partial % 16 != 0)) splits = 1;
  if (mode) mode->splits = splits;
  const long n_blocks = (long)tiles_m * tiles_n * splits;
  TW_REQUIRE(n_blocks < (1L << 30));
  // per-tile offsets are 32-bit
  TW_REQUIRE((long)BM * lda < (1L << 31));
  TW_REQUIRE(SHUF ? (long)(BN / 16) * ldw * 64 * EPF < (1L << 31) : (long)BN * ldw < (1L << 31));
  const int grid = (int)((n_blocks + 7) / 8 * 8);
  const size_t pipeline_bytes = 2 * (size_t)(BM + BN) * (KCH * 16 + 16);
  const size_t epilogue_bytes = 4 * 32 * (size_t)(32 * WN + 4) * 4;
  const size_t lds_bytes = pipeline_bytes > epilogue_bytes ? pipeline_bytes : epilogue_bytes;
  auto kernel = gemm_tiled_kernel<T, OutT, WM, WN, SHUF, GLU>;
  static bool attribute_set = false;   // per instantiation
  if (!attribute_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) return (int)e;
    attribute_set = true;
  }
  kernel<<<grid, 256, lds_bytes, stream>>>(A, lda, W, ldw, bias, residual, ldr, C, ldc, M, N, K, tiles_m,
                                           (int)n_blocks, splits, partial);
  int err = TW_LAUNCH_RESULT();
  if (err || splits == 1 || (mode && mode->leave)) return err;
  return launch_splitk_reduce<OutT>(partial, splits, bias, residual, ldr, C, ldc, M, N, stream);
}


template <typename OutT, int WM, int WN, bool GLU>
static int launch_dma(const bf16_t* A, long lda, const bf16_t* W, long ldw, const float* bias,
                      const float* residual, long ldr, OutT* C, long ldc, float* partial, long partial_bytes,
                      int M, int N, int K, int want_splits, hipStream_t stream, TiledMode* mode = nullptr) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  TW_REQUIRE(K % 32 == 0 && K >= 32 && lda % 8 == 0);
  const int tiles_m = tw_div_up(M, BM), tiles_n = tw_div_up(N, BN);
  int splits = GLU ? 1 : (want_splits > 0 ? want_splits : tiled_splits(M, N, K, 8, BM, BN));
  if (mode && mode->dry) {
    mode->splits = splits;
    return 0;
  }
  if (splits > 1 && (partial == nullptr || partial_bytes < (long)splits * M * N * 4 || (uintptr_t)partial % 16 != 0)) splits = 1;
  if (mode) mode->splits = splits;
  const long n_blocks = (long)tiles_m * tiles_n * splits;
  TW_REQUIRE(n_blocks < (1L << 30));
  // offsets within a tile's operands are 32-bit
  TW_REQUIRE((long)BM * lda * 2 < (1L << 31) && (long)(BN / 16) * ldw * 1024 < (1L << 31));
  const int grid = (int)((n_blocks + 7) / 8 * 8);
  const size_t pipeline_bytes = TW_DMA_A_SLOTS * (size_t)BM * 128 + TW_DMA_STAGES * (size_t)BN * 64;
  static_assert(TW_DMA_A_SLOTS * BM * 128 + TW_DMA_STAGES * BN * 64 <= 160 * 1024, "a workgroup has 160 KB of LDS");
  const size_t epilogue_bytes = 4 * 32 * (size_t)(32 * WN + 4) * 4;
  const size_t lds_bytes = pipeline_bytes > epilogue_bytes ? pipeline_bytes : epilogue_bytes;
  auto kernel = gemm_dma_kernel<OutT, WM, WN, GLU>;
  static bool attribute_set = false;   // per instantiation
  if (!attribute_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) return (int)e;
    attribute_set = true;
  }
  kernel<<<grid, 256, lds_bytes, stream>>>(A, lda, W, ldw, bias, residual, ldr, C, ldc, M, N, K, tiles_m,
                                           (int)n_blocks, splits, partial);
  int err = TW_LAUNCH_RESULT();
  if (err || splits == 1 || (mode && mode->leave)) return err;
  return launch_splitk_reduce<OutT>(partial, splits, bias, residual, ldr, C, ldc, M, N, stream);
}

// Which tile (1: 128x128, 2: 128x256, 3: 256x256, 4: 256x192): the one with the least estimated time,
// rounds of tiles over 256 CUs (128x128: two to a CU, so half rounds) x tile area / the rate a tile of
// that shape reaches when the chip is full (measured, relative). The estimate ranks the shapes as
// measured on the projections of 7B-class models from 256 to 16,384 rows. Larger tiles move fewer
// bytes per MFMA through the 64 B/clk vector-memory path and LDS; smaller ones waste less in the
// last round.
#ifndef TW_DMA_SHAPES
#define TW_DMA_SHAPES 0xC      /* bit s: shape s uses the direct-to-LDS kernel (at 128x128 it gains nothing) */
#endif
static const int kTileM[5] = {0, 128, 128, 256, 256}, kTileN[5] = {0, 128, 256, 256, 192};
static const double kTileRate[5] = {0, 0.76, 0.90, 1.05, 1.00};

static int choose_shape(bool big_ok, int M, int N) {
  if (!big_ok) return 1;
  int best = 1;
  double best_cost = 0;
  for (int shape = 1; shape <= 4; ++shape) {
    const long tiles = (long)tw_div_up(M, kTileM[shape]) * tw_div_up(N, kTileN[shape]);
    const double cost = (double)tw_div_up(tiles, 256) * kTileM[shape] * kTileN[shape] / kTileRate[shape];
    if (shape == 1 || cost < best_cost) {
      best = shape;
      best_cost = cost;
    }
  }
  return best;
}

// Estimated seconds of `shape` with K dealt to `splits` workgroups per tile: the rounds of workgroups
// over 256 CUs at the shape's relative rate (4.42e-13 s per unit of tile area and element of K: a
// 128x256 tile over K = 18,944 takes 295 us), plus, with splits, what splitk_reduce moves: the partial
// sums written and read, the residual and the result, at the 6.5 TB/s such just-written data streams at.
static double plan_seconds(int shape, int splits, int M, int N, int K) {
  const long tiles = (long)tw_div_up(M, kTileM[shape]) * tw_div_up(N, kTileN[shape]);
  double t = (double)tw_div_up(tiles * splits, 256) * kTileM[shape] * kTileN[shape] / kTileRate[shape] *
             ((double)K / splits) * 4.42e-13;
  if (splits > 1) t += (2.0 * splits + 2.0) * M * N * 4.0 / 6.5e12;
  return t;
}

// Shape and K ranges of a product (splits 0: the launcher's own rule for few tiles). Beside the choice
// above, 128x256 or 256x256 tiles with 2 to 8 K ranges are taken where they fill one round of CUs that whole tiles
// leave partly idle and K is long enough to pay for the reduction: the down projection of a 2,048-token
// prompt (N = 3,584, K = 18,944) has 224 tiles of 128x256 or 112 of 256x256; two K ranges of the latter
// run at the large tile's rate on 224 CUs (295 -> 265 us with the reduction).
struct TilePlan { int shape, splits; };
static TilePlan choose_plan(bool big_ok, bool glu, int M, int N, int K, int epf) {
  TilePlan plan = {choose_shape(big_ok, M, N), 0};
  if (!big_ok || glu || K % 32 != 0) return plan;
  const int own = tiled_splits(M, N, K, epf, kTileM[plan.shape], kTileN[plan.shape]);
  double best = plan_seconds(plan.shape, own, M, N, K) * 0.95;
  for (int shape = 2; shape <= 3; ++shape) {               // 128x256 and 256x256: one workgroup a CU
    const long tiles = (long)tw_div_up(M, kTileM[shape]) * tw_div_up(N, kTileN[shape]);
    for (int splits = 2; splits <= 8; ++splits) {
      if (tiles * splits > 256 || K / splits < 2048) continue;
      const double t = plan_seconds(shape, splits, M, N, K);
      if (t < best) {
        best = t;
        plan = {shape, splits};
      }
    }
  }
  return plan;
}

template <typename T, typename OutT, bool SHUF, bool GLU>
static int tiled_by_shape(int shape, const T* A, long lda, const T* W, long ldw, const float* bias,
                          const float* residual, long ldr, OutT* C, long ldc, float* partial,
                          long partial_bytes, int M, int N, int K, hipStream_t stream, TiledMode* mode = nullptr) {
  constexpr bool BIG = sizeof(T) == 2 && SHUF;
  int splits = 0;                                   // a forced shape keeps the launcher's own rule
  if (shape == 0) {
    const TilePlan plan = choose_plan(BIG, GLU, M, N, K, Elem<T>::kPerFrag);
    shape = plan.shape;
    splits = plan.splits;
  }
  if constexpr (BIG) {
    // bfloat16 and shuffled weights: the kernels that copy straight into LDS, if K allows
    if (K % 32 == 0 && K >= 32 && lda % 8 == 0) {
      if (shape == 4) return launch_dma<OutT, 4, 3, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, splits, stream, mode);
      if constexpr ((TW_DMA_SHAPES & 8) != 0)
        if (shape == 3) return launch_dma<OutT, 4, 4, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, splits, stream, mode);
      if constexpr ((TW_DMA_SHAPES & 4) != 0)
        if (shape == 2) return launch_dma<OutT, 2, 4, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, splits, stream, mode);
      if constexpr ((TW_DMA_SHAPES & 2) != 0)
        if (shape == 1) return launch_dma<OutT, 2, 2, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, splits, stream, mode);
    }
    if (shape == 3 || shape == 4)             // (K no multiple of 32: the register-staged 256x256 tile for both)
      return launch_tiled<T, OutT, 4, 4, SHUF, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, splits, stream, mode);
  }
  if (shape == 3 || shape == 4) return TW_ERR_BAD_ARGUMENT;
  if (shape == 2)
    return launch_tiled<T, OutT, 2, 4, SHUF, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, splits, stream, mode);
  return launch_tiled<T, OutT, 2, 2, SHUF, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, splits, stream, mode);
}

template <typename T, typename OutT>
static int tiled_by_layout(int shuffled, int glu, int shape, const void* A, long lda, const void* W, long ldw,
                           const float* bias, const float* residual, long ldr, void* C, long ldc, float* partial,
                           long partial_bytes, int M, int N, int K, hipStream_t stream,
                           TiledMode* mode = nullptr) {
  const T* a = (const T*)A;
  const T* w = (const T*)W;
  OutT* c = (OutT*)C;
  if (glu) {
    if constexpr (sizeof(T) == sizeof(OutT)) {
      if (shuffled) return tiled_by_shape<T, OutT, true, true>(shape, a, lda, w, ldw, bias, residual, ldr, c, ldc, partial, partial_bytes, M, N, K, stream, mode);
      return tiled_by_shape<T, OutT, false, true>(shape, a, lda, w, ldw, bias, residual, ldr, c, ldc, partial, partial_bytes, M, N, K, stream, mode);
    }
    return TW_ERR_BAD_ARGUMENT;          // the GLU form writes the input type
  }
  if (shuffled) return tiled_by_shape<T, OutT, true, false>(shape, a, lda, w, ldw, bias, residual, ldr, c, ldc, partial, partial_bytes, M, N, K, stream, mode);
  return tiled_by_shape<T, OutT, false, false>(shape, a, lda, w, ldw, bias, residual, ldr, c, ldc, partial, partial_bytes, M, N, K, stream, mode);
}

int tw_tiled_linear(int dtype, int out_f32, int shuffled, int glu, int shape, const void* A, long lda,
                    const void* W, long ldw, const float* bias, const float* residual, long ldr, void* C,
                    long ldc, float* partial, long partial_bytes, int M, int N, int K, hipStream_t stream) {
  TW_REQUIRE(shape >= 0 && shape <= 4);
  if (dtype == TW_DTYPE_F32)
    return tiled_by_layout<float, float>(shuffled, glu, shape, A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  if (dtype != TW_DTYPE_BF16) return TW_ERR_BAD_ARGUMENT;
  if (out_f32)
    return tiled_by_layout<bf16_t, float>(shuffled, glu, shape, A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  return tiled_by_layout<bf16_t, bf16_t>(shuffled, glu, shape, A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
}

// K ranges the tiled kernels would use for this product (1: no split).
int tw_tiled_partial_splits(int dtype, int shuffled, long lda, int M, int N, int K) {
  TiledMode mode;
  mode.dry = true;
  int err;
  if (dtype == TW_DTYPE_F32)
    err = tiled_by_layout<float, float>(shuffled, 0, 0, nullptr, lda, nullptr, K, nullptr, nullptr, 0, nullptr, N, nullptr, 0, M, N, K, nullptr, &mode);
  else if (dtype == TW_DTYPE_BF16)
    err = tiled_by_layout<bf16_t, float>(shuffled, 0, 0, nullptr, lda, nullptr, K, nullptr, nullptr, 0, nullptr, N, nullptr, 0, M, N, K, nullptr, &mode);
  else
    return 0;
  return err ? 0 : mode.splits;
}

// partial[s][M][N] (float32) = A[:, K range s] W[:, K range s]^T for the ranges the tiled kernels choose;
// no reduction. *splits_used tells how many ranges there are (1: partial[0] is the product itself).
int tw_tiled_partials(int dtype, int shuffled, const void* A, long lda, const void* W, long ldw, float* partial,
                      long partial_bytes, int M, int N, int K, int* splits_used, hipStream_t stream) {
  TW_REQUIRE(partial != nullptr && (uintptr_t)partial % 16 == 0 && partial_bytes >= (long)M * N * 4);
  TiledMode mode;
  mode.leave = true;
  int err;
  if (dtype == TW_DTYPE_F32)
    err = tiled_by_layout<float, float>(shuffled, 0, 0, A, lda, W, ldw, nullptr, nullptr, 0, partial, N, partial, partial_bytes, M, N, K, stream, &mode);
  else if (dtype == TW_DTYPE_BF16)
    err = tiled_by_layout<bf16_t, float>(shuffled, 0, 0, A, lda, W, ldw, nullptr, nullptr, 0, partial, N, partial, partial_bytes, M, N, K, stream, &mode);
  else
    return TW_ERR_BAD_ARGUMENT;
  if (splits_used) *splits_used = mode.splits;
  return err;
}

long tw_tiled_workspace_bytes(int dtype, int rows, int N, int K) {
  const int epf = dtype == TW_DTYPE_F32 ? 4 : 8;
  // enough for whichever kernel runs: the 128x128 tiles' own rule, or the plan for shuffled bfloat16 weights
  const int splits = tiled_splits(rows, N, K, epf, 128, 128);
  long bytes = splits > 1 ? (long)splits * rows * N * 4 : 0;
  if (dtype == TW_DTYPE_BF16) {
    const TilePlan plan = choose_plan(true, false, rows, N, K, epf);
    const int s = plan.splits > 0 ? plan.splits : tiled_splits(rows, N, K, epf, kTileM[plan.shape], kTileN[plan.shape]);
    if (s > 1 && (long)s * rows * N * 4 > bytes) bytes = (long)s * rows * N * 4;
  }
  return bytes;
}
