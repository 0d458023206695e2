// Linear layers: C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) (+ residual[M, N]).
// A and W are both contiguous along K (the checkpoint's [out, in] layout), in
// float32 or bfloat16; accumulation is float32 on the MFMA units (true float32
// MFMA for float32 inputs, no reduced-precision matrix mode). Three kernels:
//   gemm_tiled      - many rows (prompt portions): LDS-staged 32x32 MFMA tiles
//   gemm_skinny_lds - few rows (decode): weights streamed once from HBM straight
//                     into 16x16 MFMA fragments, split over K when N is small
//   gemm_generic    - any K (rows not 16-byte aligned): one output per thread
//
// Weight layouts. Row-major [N][K] as in the checkpoint, or SHUFFLED (an exact permutation,
// zero padded): blocks of 16 rows x 4 sixteen-byte chunks stored in the order the MFMA units
// read them, [N/16][K/(4*EPF)][chunk 0..3][row 0..15][EPF]. Element (n, k) is at
//   ((n/16 * k_steps + (k/EPF)/4) * 64 + ((k/EPF)%4) * 16 + n%16) * EPF + k%EPF.
// A wave's load of one block is 1 KB of consecutive memory: the decode kernel streams weights
// as whole cache lines past the caches (non-temporal), the tiled kernel copies blocks.
//
// GLU (gated linear unit) form: the N rows of W are the gate and up projections interleaved in
// blocks of 16 rows (gate rows 16j.., then up rows 16j.., for j = 0, 1, ...). The kernels form
// C[M, N/2][.., 16j + i] = silu(gate_j[i]) * up_j[i] in their epilogues, in float32 from the
// accumulators, so the [M, N] intermediate never reaches memory.
#include <type_traits>
#include "tw_common.h"
#include "gemm_shared.h"

// element offset of (row n, 16-byte chunk c) in the shuffled layout
__device__ __forceinline__ size_t tw_shuffled_chunk(int n, int c, int k_steps, int epf) {
  return ((size_t)((size_t)(n >> 4) * k_steps + (c >> 2)) * 64 + (c & 3) * 16 + (n & 15)) * epf;
}

// =====================================================================================
// Skinny kernel (M <= 16*MT rows), workgroup-cooperative. The WAVES (4, or 2) waves of a workgroup own
// neighbouring tiles of 16 output columns and the SAME K range. Per stage of U
// MFMA steps the workgroup copies the activations' K slice [16*MT rows][U*64 B]
// to LDS once (instead of every wave reading it from L2); each wave streams its
// own 16 weight rows from global memory into registers (every weight byte is read by exactly
// one wave). Two stages of weights in flight. splits == 1: the epilogue runs here. splits > 1: float32
// partial sums go to partial[split][M][N] and splitk_reduce_kernel (or the caller's next
// kernel) adds them, always in the same order, so results do not depend on timing.
// =====================================================================================
#define TW_XROW(U) ((U) * 64 + 32)          /* LDS bytes per activation row of a stage, padded: 32 * an odd number (see tw_lds_swz4) */

// PARTIAL: always write float32 partial sums partial[split][M][N] (splits >= 1), no epilogue.
// SHUF: W is in the shuffled layout (ldw = its k_steps): every weight load is 1 KB of consecutive
// memory, needs no predicate (the layout is zero padded) and bypasses the caches.
// GLU (splits == 1 only): the workgroup's tiles are gate, up(, gate, up); C gets half as many columns.
// WAVES = 2 halves the workgroups' size and doubles their number: used where that spreads them more
// evenly over the CUs (the kernel's time is that of the fullest CU).
template <typename T, typename OutT, int MT, int U, int WAVES, bool PARTIAL, bool SHUF, bool GLU>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_lds_kernel(const T* __restrict__ A, long lda,
                                                              const T* __restrict__ W, long ldw,
                                                              const float* __restrict__ bias,
                                                              const float* residual, long ldr, OutT* C,
                                                              long ldc, float* __restrict__ partial, int M,
                                                              int N, int K, int n_groups, int splits) {
  typedef typename Elem<T>::Frag Frag;
  constexpr int EPF = Elem<T>::kPerFrag;
  constexpr int XROW = TW_XROW(U);
  constexpr int XSTAGE = MT * 16 * XROW;
  constexpr int THREADS = WAVES * 64;
  constexpr int XLOADS = MT * U / WAVES;               // activation fragments per thread per stage
  static_assert(U % 4 == 0 && (WAVES == 4 || WAVES == 2), "a stage is copied by all threads in whole rounds");
  __shared__ __attribute__((aligned(16))) char lds[2 * XSTAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int group = blockIdx.x % n_groups, split = blockIdx.x / n_groups;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = group * (16 * WAVES) + wave * 16;

  const int chunks = K / EPF;
  const int steps = (chunks + 3) / 4;
  const int steps_per_split = (steps + splits - 1) / splits;
  const int step_begin = split * steps_per_split;
  const int step_end = min(steps, step_begin + steps_per_split);
  const int n_stages = step_end > step_begin ? (step_end - step_begin + U - 1) / U : 0;

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const T* w_row = SHUF ? W + ((size_t)min(n0 / 16, (N + 15) / 16 - 1) * ldw * 64 + lane) * EPF
                        : W + (size_t)min(n0 + r, N - 1) * ldw;
  // this thread's share of the activation slice: fragment f = i*THREADS + tid -> (row f / (4U), chunk f % (4U))
  const T* x_src[XLOADS];
  int x_dst[XLOADS], x_chunk[XLOADS];
#pragma unroll
  for (int i = 0; i < XLOADS; ++i) {
    const int f = i * THREADS + tid, row = f / (4 * U), c = f % (4 * U);
    x_src[i] = A + (size_t)min(row, M - 1) * lda;
    x_chunk[i] = c;
    x_dst[i] = row * XROW + c * 16;
  }

  // Loads carry no predicate: addresses are clamped to the last valid step or chunk (always inside
  // the matrix), and activation chunks outside this workgroup's K range are replaced by zeros on
  // their way to LDS, so whatever weight was read beside them adds nothing. Without conditional
  // loads the compiler's wait counts are exact, which the order of the pipeline below relies on.
  Frag wf[2][U], xg[XLOADS];
  const int chunk_end = min(step_end * 4, chunks);
  auto load_w = [&](const int buf, int s0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (SHUF)
        wf[buf][u] = tw_load_frag_stream(w_row + (size_t)min(s0 + u, steps - 1) * 64 * EPF);
      else
        wf[buf][u] = tw_load_frag(w_row + (size_t)min((s0 + u) * 4 + g, chunks - 1) * EPF);
    }
  };
  auto load_x = [&](int s0) {
#pragma unroll
    for (int i = 0; i < XLOADS; ++i)
      xg[i] = tw_load_frag(x_src[i] + (size_t)min(s0 * 4 + x_chunk[i], chunks - 1) * EPF);
  };
  auto store_x = [&](int buf, int s0) {
#pragma unroll
    for (int i = 0; i < XLOADS; ++i)
      *reinterpret_cast<Frag*>(lds + buf * XSTAGE + x_dst[i]) = s0 * 4 + x_chunk[i] < chunk_end ? xg[i] : Elem<T>::zero();
  };
  auto multiply = [&](const int buf) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const Frag xf = *reinterpret_cast<const Frag*>(lds + buf * XSTAGE + (mt * 16 + r) * XROW + (u * 4 + g) * 16);
        tw_mma16(acc[mt], wf[buf][u], xf);
      }
  };
  // Two stages i, i + 1 (i even: stage i has its weights in register set 0 and its activations in
  // LDS buffer 0). Per stage: request the next stage's activations, multiply this stage, request
  // the weights of the stage after next into the registers just used, then move the activations to
  // LDS. Loads return in order, so the wait for the activations leaves the newest weight loads in
  // flight: a wave that stalls there has one to two stages of weights on their way.
  auto stage_pair = [&](int i, auto more1, auto more2, auto more3) {
    const int s0 = step_begin + i * U;
    if (more1) load_x(s0 + U);
    __builtin_amdgcn_sched_barrier(0);           // the compiler would sink the loads below the waits
    multiply(0);
    if (more2) load_w(0, s0 + 2 * U);
    __builtin_amdgcn_sched_barrier(0);
    if (more1) store_x(1, s0 + U);
    __syncthreads();
    if (!more1) return;
    if (more2) load_x(s0 + 2 * U);
    __builtin_amdgcn_sched_barrier(0);
    multiply(1);
    if (more3) load_w(1, s0 + 3 * U);
    __builtin_amdgcn_sched_barrier(0);
    if (more2) store_x(0, s0 + 2 * U);
    __syncthreads();
  };

  if (n_stages > 0) {
    load_x(step_begin);
    load_w(0, step_begin);
    if (n_stages > 1) load_w(1, step_begin + U);
    store_x(0, step_begin);
    __syncthreads();
    int i = 0;
    for (; i + 3 < n_stages; i += 2) stage_pair(i, std::true_type{}, std::true_type{}, std::true_type{});
    for (; i < n_stages; i += 2) stage_pair(i, i + 1 < n_stages, i + 2 < n_stages, i + 3 < n_stages);
  }

  // acc[mt][j] = sum_k W[n0 + 4g + j][k] * A[16 mt + r][k]
  if (GLU) {
    // the waves swap their tiles through LDS (every wave is past its last LDS read: the loop
    // ends with a barrier), then each thread forms outputs from a (gate, up) pair
    constexpr int GROW = 17;                                  // floats per staged row, padded
    static_assert(WAVES * MT * 16 * GROW * 4 <= 2 * XSTAGE, "the GLU exchange fits the pipeline's LDS");
    float* ex = reinterpret_cast<float*>(lds);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = n0 + 4 * g + j;
        ex[(wave * MT * 16 + mt * 16 + r) * GROW + 4 * g + j] = acc[mt][j] + (bias && col < N ? bias[col] : 0.f);
      }
    __syncthreads();
    constexpr int OUT_COLS = 8 * WAVES;                       // output columns of the workgroup
    for (int o = tid; o < MT * 16 * OUT_COLS; o += THREADS) {
      const int row = o / OUT_COLS, c = o % OUT_COLS, pair = c >> 4, i = c & 15;
      const int col = group * OUT_COLS + c;                   // output column
      if (row >= M || col >= N / 2) continue;
      const float gv = ex[((2 * pair) * MT * 16 + row) * GROW + i];
      const float uv = ex[((2 * pair + 1) * MT * 16 + row) * GROW + i];
      C[(size_t)row * ldc + col] = tw_from_float<OutT>(tw_silu(gv) * uv);
    }
    return;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = mt * 16 + r;
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + 4 * g + j;
      if (col >= N) continue;
      if (PARTIAL || splits > 1) {
        partial[((size_t)split * M + row) * N + col] = acc[mt][j];
      } else {
        float v = acc[mt][j] + (bias ? bias[col] : 0.f);
        if (residual) v += residual[(size_t)row * ldr + col];
        C[(size_t)row * ldc + col] = tw_from_float<OutT>(v);
      }
    }
  }
}

// =====================================================================================
// Streaming kernel with ONE workgroup per CU (shuffled weights; the launcher uses it above 16 rows).
//
// The kernel above deals whole workgroups of four column tiles to the CUs, a few hundred of them, and every
// workgroup stages its own copy of the activations, which at 64 rows are as many bytes from L2 as the
// weights are from HBM. Here the grid is one workgroup per CU and the 16-column tiles (or gate/up pairs
// of them) are dealt to the workgroups as evenly as whole tiles allow, K ranges first where one range
// would leave CUs idle. A workgroup is TW_CU_WAVES waves: up to TW_CU_MAX_COMPUTE of them take one tile
// each per round (several rounds if the workgroup has more tiles), the others only help with the copies.
// EVERY wave copies its share of the activations' K slice of each stage from global memory straight into
// LDS (`global_load_lds_dwordx4`: no staging registers, no LDS write instructions, one copy per CU instead
// of one per four tiles; the copies of a stage are dealt to all waves because a wave's copies go out one
// after the other). Compute waves stream their own 16 weight rows into registers, TW_CU_NBUF - 1 stages
// ahead, and multiply out of LDS.
//
// LDS layout of a stage: MT * U blocks of 1 KB, block (mt, u) = rows 16 mt .. 16 mt + 15, the four
// 16-byte chunks of k-step u. Slot l of a block holds row l / 4, chunk (l % 4) ^ (row / 4 % 4): four
// neighbouring lanes fetch 64 consecutive bytes, and the 16 lanes that read one chunk of 16 rows meet
// 16 different bank groups. Chunks outside the workgroup's K range are copied from a chunk of zeros,
// so whatever weight is read beside them adds nothing; rows past M are clamped (never stored).
// =====================================================================================
#ifndef TW_CU_NBUF
#define TW_CU_NBUF 4
#endif
#ifndef TW_CU_U
#define TW_CU_U 4
#endif
#ifndef TW_CU_WAVES
#define TW_CU_WAVES 16
#endif
#ifndef TW_CU_MAX_COMPUTE
#define TW_CU_MAX_COMPUTE 14
#endif
/* more than half a CU's LDS (never two of these workgroups on one CU), room for the stages of 64 rows, and 1 KB
   where copies that a wave has no block for are dumped */
#define TW_CU_STAGES_BYTES (TW_CU_NBUF * TW_CU_U * 4 * 1024)
#define TW_CU_LDS_BYTES ((TW_CU_STAGES_BYTES + 1024) > 84 * 1024 ? (TW_CU_STAGES_BYTES + 1024) : 84 * 1024)

__device__ __attribute__((aligned(16))) const uint32_t tw_zero_chunk[4] = {0u, 0u, 0u, 0u};

typedef __attribute__((address_space(3))) void* tw_lds_dst;

template <typename T, typename OutT, int MT, bool PARTIAL, bool GLU>
__global__ __launch_bounds__(TW_CU_WAVES * 64) void gemm_stream_cu_kernel(
    const T* __restrict__ A, long lda, const T* __restrict__ W, long ldw, const float* __restrict__ bias,
    const float* residual, long ldr, OutT* C, long ldc, float* __restrict__ partial, int M, int N, int K,
    int splits, int wgs_per_split, int compute_waves, int steps_per_split, int vec) {
  typedef typename Elem<T>::Frag Frag;
  constexpr int EPF = Elem<T>::kPerFrag, U = TW_CU_U, NBUF = TW_CU_NBUF, WAVES = TW_CU_WAVES;
  constexpr int BLOCKS = MT * U;                       // 1 KB blocks of activations per stage
  constexpr int XSTAGE = BLOCKS * 1024;
  constexpr int XD = (BLOCKS + WAVES - 1) / WAVES;     // copies per wave and stage
  static_assert(NBUF * XSTAGE + 1024 <= TW_CU_LDS_BYTES && NBUF >= 3, "stage layout");
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = blockIdx.x % wgs_per_split, split = blockIdx.x / wgs_per_split;
  // this workgroup's tiles of 16 columns: [t0, t1), whole gate/up pairs for GLU
  constexpr int UW = GLU ? 2 : 1;
  const long units = GLU ? N / 32 : (N + 15) / 16;
  const int t0 = (int)(units * j / wgs_per_split) * UW, t1 = (int)(units * (j + 1) / wgs_per_split) * UW;
  const int last_block = (N + 15) / 16 - 1;
  // this workgroup's K range, in k-steps of four 16-byte chunks
  const int chunks = K / EPF, steps = (chunks + 3) / 4;
  const int step_begin = min(steps, split * steps_per_split), step_end = min(steps, step_begin + steps_per_split);
  const int n_stages = (step_end - step_begin + U - 1) / U;
  const int chunk_end = min(step_end * 4, chunks);
  const int r = lane & 15, g = lane >> 4;

#define TW_CU_WAIT(n) asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory")
#define TW_CU_BARRIER()                   \
  do {                                    \
    __builtin_amdgcn_s_barrier();         \
    asm volatile("" ::: "memory");        \
  } while (0)
  // Wait until at most `n` of this wave's loads and copies are in flight (they finish in the order they
  // were issued). The count is an immediate of the instruction, hence the cases.
  auto wait_for = [&](auto n) {
    constexpr int N_ = decltype(n)::value;
    if constexpr (N_ == 2) TW_CU_WAIT(2);
    else if constexpr (N_ == 4) TW_CU_WAIT(4);
    else if constexpr (N_ == 6) TW_CU_WAIT(6);
    else if constexpr (N_ == 8) TW_CU_WAIT(8);
    else if constexpr (N_ == 10) TW_CU_WAIT(10);
    else if constexpr (N_ == 12) TW_CU_WAIT(12);
    else if constexpr (N_ == 14) TW_CU_WAIT(14);
    else if constexpr (N_ == 16) TW_CU_WAIT(16);
    else if constexpr (N_ == 18) TW_CU_WAIT(18);
    else if constexpr (N_ == 20) TW_CU_WAIT(20);
    else if constexpr (N_ == 24) TW_CU_WAIT(24);
    else TW_CU_WAIT(0);
  };

  // ---- this wave's share of the activation copies: blocks wave, wave + WAVES, ... of every stage ----
  const int row16 = lane >> 2, cswz = (lane & 3) ^ tw_lds_swz4(row16);
  const T* x_row[XD];
  int x_chunk[XD], x_dst[XD];
#pragma unroll
  for (int q = 0; q < XD; ++q) {
    const int b = wave + WAVES * q;
    const bool mine = b < BLOCKS;                          // else: a copy of zeros into the dump area
    const int mt = mine ? b / U : 0, u = mine ? b % U : 0;
    x_row[q] = A + (size_t)min(mt * 16 + row16, M - 1) * lda;
    x_chunk[q] = mine ? u * 4 + cswz : (1 << 28);          // (a chunk far outside every K range)
    x_dst[q] = mine ? b * 1024 : -1;
  }
  auto copy_x = [&](int stage, const int buf) {
    const int c0 = (step_begin + stage * U) * 4;
#pragma unroll
    for (int q = 0; q < XD; ++q) {
      const int c = c0 + x_chunk[q];
      const T* src = c < chunk_end ? x_row[q] + (size_t)c * EPF : reinterpret_cast<const T*>(tw_zero_chunk);
      char* dst = x_dst[q] >= 0 ? lds + buf * XSTAGE + x_dst[q] : lds + NBUF * XSTAGE;
      // (the cast matters: handed a pointer whose type depends on a template parameter, the host pass drops
      // the kernel's definition without a word and the library no longer links)
      __builtin_amdgcn_global_load_lds((const void*)src, (tw_lds_dst)dst, 16, 0, 0);
    }
  };

  for (int first = t0; first < t1; first += compute_waves) {       // rounds: the same for every wave
    const int tile = first + wave;
    if (wave >= compute_waves || tile >= t1) {
      // ---- a wave without a tile in this round: copies only ------------------------------------------
      // stage i's copies have landed once at most the NBUF - 2 newer stages' are in flight
#pragma unroll
      for (int b = 0; b < NBUF - 1; ++b) copy_x(b, b);
      auto stage_h = [&](int i, const int buf) {
        wait_for(std::integral_constant<int, XD * (NBUF - 2)>{});
        TW_CU_BARRIER();                                    // stage i is there for every wave; every wave is past stage i - 1
        copy_x(i + NBUF - 1, (buf + NBUF - 1) % NBUF);      // into the stage that was read last (past the end: zeros)
      };
      int i = 0;
      for (; i + NBUF <= n_stages; i += NBUF) {
#pragma unroll
        for (int b = 0; b < NBUF; ++b) stage_h(i + b, b);
      }
#pragma unroll
      for (int b = 0; b < NBUF; ++b)
        if (i + b < n_stages) stage_h(i + b, b);
      TW_CU_WAIT(0);                                        // no copy lands after the loop
      TW_CU_BARRIER();                                      // (E1)
      if (GLU) {
        TW_CU_BARRIER();                                    // (E2)
        TW_CU_BARRIER();                                    // (E3)
      }
      continue;
    }
    // ---- a wave with a tile of 16 columns --------------------------------------------------------------
    const T* w_row = W + ((size_t)min(tile, last_block) * ldw * 64 + lane) * EPF + (size_t)step_begin * 64 * EPF;
    const int slot = (r * 4 + (g ^ tw_lds_swz4(r))) * 16;
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    Frag wf[NBUF][U];
    const int last_step = steps - 1 - step_begin;           // (relative to this workgroup's first k-step)
    auto load_w = [&](int stage, const int buf) {
#pragma unroll
      for (int u = 0; u < U; ++u)
        wf[buf][u] = tw_load_frag_stream(w_row + (size_t)min(stage * U + u, last_step) * (64 * EPF));
    };
    auto multiply = [&](const int buf) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        Frag xf[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          xf[mt] = *reinterpret_cast<const Frag*>(lds + buf * XSTAGE + (mt * U + u) * 1024 + slot);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) tw_mma16(acc[mt], wf[buf][u], xf[mt]);
        // one k-step's fragments at a time: the other waves of the CU cover the LDS latency, and the registers
        // that reading a whole stage ahead would take are what the weights in flight need
        if (MT > 1) __builtin_amdgcn_sched_barrier(0);
      }
    };
    // Stage i: wait for this wave's copies of stage i, meet the others (stage i's activations are in LDS,
    // stage i - 1's are read), ask for the weights and copies of stage i + NBUF - 1, multiply. In the main
    // loop every stage issues U loads and XD copies, so "the NBUF - 2 newer stages may be in flight" is a
    // count; near the end the stages after the last one issue copies (of zeros) but no loads.
    auto stage_c = [&](int i, const int buf, auto main) {
      static_assert(NBUF == 4 || NBUF == 3, "the cases below");
      const int newer = main ? NBUF - 2 : min(max(n_stages - 1 - i, 0), NBUF - 2);   // newer stages with loads
      if (newer == NBUF - 2) wait_for(std::integral_constant<int, (U + XD) * (NBUF - 2)>{});
      else if (newer == 1) wait_for(std::integral_constant<int, U + XD * (NBUF - 2)>{});
      else wait_for(std::integral_constant<int, XD * (NBUF - 2)>{});
      TW_CU_BARRIER();
      if (main || i + NBUF - 1 < n_stages) load_w(i + NBUF - 1, (buf + NBUF - 1) % NBUF);
      copy_x(i + NBUF - 1, (buf + NBUF - 1) % NBUF);
      __builtin_amdgcn_sched_barrier(0);                    // (loads and copies go out before the multiplies, not after)
      multiply(buf);
    };
#pragma unroll
    for (int b = 0; b < NBUF - 1; ++b) {
      if (b < n_stages) load_w(b, b);
      copy_x(b, b);
    }
    int i = 0;
    if (n_stages >= NBUF - 1)                               // (else the prologue issued fewer loads than the counts assume)
      for (; i + 2 * NBUF - 1 <= n_stages; i += NBUF) {     // every load of these stages names a stage that exists
#pragma unroll
        for (int b = 0; b < NBUF; ++b) stage_c(i + b, b, std::true_type{});
      }
    for (; i < n_stages; i += NBUF) {
#pragma unroll
      for (int b = 0; b < NBUF; ++b)
        if (i + b < n_stages) stage_c(i + b, b, std::false_type{});
    }
    TW_CU_WAIT(0);                                          // no copy lands after the loop
    TW_CU_BARRIER();                                        // (E1) every wave is past its last LDS read

    // acc[mt][e] = sum_k W[16 tile + 4g + e][k] * A[16 mt + r][k]
    const int col0 = tile * 16 + 4 * g;
    if (GLU) {
      // the two waves of a gate/up pair swap their tiles through LDS; each thread then forms outputs
      constexpr int GROW = 17;
      float* ex = reinterpret_cast<float*>(lds);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          ex[((wave * MT + mt) * 16 + r) * GROW + 4 * g + e] = acc[mt][e] + (bias && col0 + e < N ? bias[col0 + e] : 0.f);
      TW_CU_BARRIER();                                      // (E2)
      {
        const int gate_wave = wave & ~1;
        const int out0 = ((first + gate_wave) >> 1) * 16;   // first output column of the pair
        for (int o = (wave & 1) * 64 + lane; o < MT * 16 * 16; o += 128) {
          const int row = o >> 4, c = o & 15;
          if (row >= M || out0 + c >= N / 2) continue;
          const float gv = ex[(gate_wave * MT * 16 + row) * GROW + c];
          const float uv = ex[((gate_wave + 1) * MT * 16 + row) * GROW + c];
          C[(size_t)row * ldc + out0 + c] = tw_from_float<OutT>(tw_silu(gv) * uv);
        }
      }
      TW_CU_WAIT(0);
      TW_CU_BARRIER();                                      // (E3) the exchange area is free for the next round's copies
      continue;
    }
    {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int row = mt * 16 + r;
        if (row >= M || col0 >= N) continue;
        if (PARTIAL || splits > 1) {
          float* dst = partial + ((size_t)split * M + row) * N + col0;
          if (vec) {
            *reinterpret_cast<f32x4*>(dst) = acc[mt];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (col0 + e < N) dst[e] = acc[mt][e];
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (col0 + e >= N) continue;
            float v = acc[mt][e] + (bias ? bias[col0 + e] : 0.f);
            if (residual) v += residual[(size_t)row * ldr + col0 + e];
            C[(size_t)row * ldc + col0 + e] = tw_from_float<OutT>(v);
          }
        }
      }
    }
    TW_CU_WAIT(0);        // stores and loads are counted together but finish apart: start the next round from zero
  }
#undef TW_CU_WAIT
#undef TW_CU_BARRIER
}

// =====================================================================================
// Generic kernel: any K. One thread per output element, float32 accumulation.
// =====================================================================================
template <typename T>
__device__ __forceinline__ float tw_generic_dot(const T* a, const T* W, long ldw, int col, int K, int shuffled) {
  constexpr int EPF = Elem<T>::kPerFrag;
  float v = 0.f;
  if (shuffled) {
    for (int k = 0; k < K; ++k)
      v = fmaf(tw_to_float(a[k]), tw_to_float(W[tw_shuffled_chunk(col, k / EPF, (int)ldw, EPF) + k % EPF]), v);
  } else {
    const T* w = W + (size_t)col * ldw;
    for (int k = 0; k < K; ++k) v = fmaf(tw_to_float(a[k]), tw_to_float(w[k]), v);
  }
  return v;
}

// glu: C has N / 2 columns (see the top of the file)
template <typename T, typename OutT>
__global__ void gemm_generic_kernel(const T* __restrict__ A, long lda, const T* __restrict__ W, long ldw,
                                    const float* __restrict__ bias, const float* residual, long ldr,
                                    OutT* C, long ldc, int M, int N, int K, int shuffled, int glu) {
  const int n_out = glu ? N / 2 : N;
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)M * n_out) return;
  const int row = (int)(i / n_out), col = (int)(i % n_out);
  const T* a = A + (size_t)row * lda;
  if (glu) {
    const int gate = (col / 16) * 32 + col % 16, up = gate + 16;
    const float gv = tw_generic_dot(a, W, ldw, gate, K, shuffled) + (bias ? bias[gate] : 0.f);
    const float uv = tw_generic_dot(a, W, ldw, up, K, shuffled) + (bias ? bias[up] : 0.f);
    C[(size_t)row * ldc + col] = tw_from_float<OutT>(tw_silu(gv) * uv);
    return;
  }
  float v = tw_generic_dot(a, W, ldw, col, K, shuffled);
  if (bias) v += bias[col];
  if (residual) v += residual[(size_t)row * ldr + col];
  C[(size_t)row * ldc + col] = tw_from_float<OutT>(v);
}

// =====================================================================================
// Host side
// =====================================================================================
// How many K ranges the skinny kernel uses for an [N, K] weight: as many as keep the workgroups at or
// under two for each of the 256 CUs (all resident at once and evenly spread: with 560 workgroups, a few
// over that, some CUs hold three and the kernel takes 10-15 % longer than with 504), each range at
// least 16 MFMA steps long. The choice depends on N and K only, never on the rows of a batch.
static int skinny_lds_splits(int N, int K, int epf) {
  const int groups = tw_div_up(N, 64);
  const int steps = tw_div_up(K / epf, 4);
  int splits = 512 / groups;
  const int max_by_k = steps / 16 > 0 ? steps / 16 : 1;
  if (splits > max_by_k) splits = max_by_k;
  if (splits > 16) splits = 16;
  return splits < 1 ? 1 : splits;
}

// ---- the kernel with one workgroup per CU: how its work is dealt ---------------------------------
static int cu_count() {
  static int cus = 0;                        // (the same for every device of a box)
  if (cus == 0) {
    int device = 0, n = 0;
    if (hipGetDevice(&device) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

struct CuPlan { int splits, wgs_per_split, compute_waves, steps_per_split; };

// K ranges, workgroups per range and compute waves per workgroup for MT row tiles against an [N, K] weight.
// Every candidate number of ranges is priced by the bytes its fullest CU streams (whole tiles, K ranges
// rounded up to whole stages), more where a CU would have few waves to keep loads in flight, plus the
// start of each round and, with more than one range, the partial sums written and read again; the
// cheapest wins. Depends on the row tiles, N and K only, never on the rows of a batch within a tile.
static CuPlan cu_plan(int MT, int N, int K, int epf, bool glu, bool may_split) {
  const int cus = cu_count();
  const int uw = glu ? 2 : 1;
  const long units = glu ? N / 32 : tw_div_up(N, 16);
  const int steps = tw_div_up(K / epf, 4);
  int most = may_split && !glu ? steps / 8 : 1;
  if (most > 16) most = 16;
  if (most < 1) most = 1;
  CuPlan best = {1, 1, 1, steps};
  double best_cost = 0;
  for (int want = 1; want <= most; ++want) {
    const int sps = tw_div_up(tw_div_up(steps, want), TW_CU_U) * TW_CU_U;
    const int splits = tw_div_up(steps, sps);
    if (splits != want && want > 1) continue;                       // (a count that rounding maps onto another one)
    long wgs = cus / splits;
    if (wgs > units) wgs = units;
    if (wgs < 1) wgs = 1;
    const long tiles = tw_div_up(units, wgs) * uw;                  // of the fullest workgroup
    const int rounds = tw_div_up(tiles, TW_CU_MAX_COMPUTE);
    int waves = tw_div_up(tiles, rounds);
    if (glu && waves % 2) ++waves;
    const double stream = (double)tiles * sps * 1024.0 / (waves >= 8 ? 1.0 : waves / 8.0);
    const double partial = splits > 1 || !glu ? 2.0 * splits * (16.0 * MT) * N * 4.0 / cus : 0.0;
    const double cost = stream + rounds * 37000.0 + (splits > 1 ? partial : 0.0);
    if (want == 1 || cost < best_cost) {
      best = {splits, (int)wgs, waves, sps};
      best_cost = cost;
    }
  }
  return best;
}

// Bytes of split-K scratch tw_linear can use for up to max_rows rows (0: none needed).
extern "C" long tw_linear_workspace_bytes(int dtype, int max_rows, int N, int K) {
  const int epf = dtype == TW_DTYPE_F32 ? 4 : 8;
  if (K % epf) return 0;
  const int rows = max_rows < 64 ? max_rows : 64;
  int splits = skinny_lds_splits(N, K, epf);
  for (int mt = 1; mt <= tw_div_up(rows, 16); ++mt) {          // whichever streaming kernel runs for these rows
    const int s = cu_plan(mt, N, K, epf, false, true).splits;
    if (s > splits) splits = s;
  }
  long bytes = splits > 1 ? (long)splits * rows * N * 4 : 0;
  if (max_rows > 64) {
    const long tiled = tw_tiled_workspace_bytes(dtype, max_rows, N, K);
    if (tiled > bytes) bytes = tiled;
  }
  return bytes;
}

// The fullest CU's share of `workgroups` spread over 256 CUs, relative to an even spread.
static double cu_imbalance(long workgroups) {
  return workgroups <= 256 ? 1.0 : (double)tw_div_up(workgroups, 256) * 256.0 / (double)workgroups;
}

template <typename T, typename OutT, int MT, bool PARTIAL, bool SHUF, bool GLU>
static int launch_skinny_lds(const T* A, long lda, const T* W, long ldw, const float* bias,
                             const float* residual, long ldr, OutT* C, long ldc, float* partial,
                             long partial_bytes, int M, int N, int K, hipStream_t stream) {
  constexpr int EPF = Elem<T>::kPerFrag;
  constexpr int U = MT == 1 ? 8 : 4;
  int splits = GLU ? 1 : skinny_lds_splits(N, K, EPF);
  if (PARTIAL) {
    TW_REQUIRE(partial != nullptr && partial_bytes >= (long)splits * M * N * 4);
  } else if (splits > 1 && (partial == nullptr || partial_bytes < (long)splits * M * N * 4)) {
    splits = 1;
  }
  // One K range and at most 16 rows (the gated projection of a decode step, the head): workgroups of two
  // waves where twice as many of them lie more evenly on the CUs (N = 37,888: 592 workgroups are 2.3 a CU,
  // three on some; 1,184 are 4.6, five on some). With more rows every workgroup stages its own copy of
  // the activations, so the larger workgroups stay.
  if constexpr (MT == 1 && !PARTIAL) {
    if (splits == 1 && cu_imbalance(tw_div_up(N, 32)) < cu_imbalance(tw_div_up(N, 64)) - 0.03) {
      const int groups = tw_div_up(N, 32);
      gemm_skinny_lds_kernel<T, OutT, MT, U, 2, PARTIAL, SHUF, GLU><<<groups, 128, 0, stream>>>(
          A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, M, N, K, groups, 1);
      return TW_LAUNCH_RESULT();
    }
  }
  const int groups = tw_div_up(N, 64);
  gemm_skinny_lds_kernel<T, OutT, MT, U, 4, PARTIAL, SHUF, GLU><<<groups * splits, 256, 0, stream>>>(
      A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, M, N, K, groups, splits);
  int err = TW_LAUNCH_RESULT();
  if (err || splits == 1 || PARTIAL) return err;
  return launch_splitk_reduce<OutT>(partial, splits, bias, residual, ldr, C, ldc, M, N, stream);
}

template <typename T, typename OutT, int MT, bool PARTIAL, bool GLU>
static int launch_stream_cu_mt(const T* A, long lda, const T* W, long ldw, const float* bias, const float* residual,
                               long ldr, OutT* C, long ldc, float* partial, long partial_bytes, int M, int N, int K,
                               hipStream_t stream) {
  constexpr int EPF = Elem<T>::kPerFrag;
  const bool room = partial != nullptr;
  CuPlan plan = cu_plan(MT, N, K, EPF, GLU, PARTIAL || room);
  if (PARTIAL) {
    TW_REQUIRE(partial != nullptr && partial_bytes >= (long)plan.splits * M * N * 4);
  } else if (plan.splits > 1 && partial_bytes < (long)plan.splits * M * N * 4) {
    plan = cu_plan(MT, N, K, EPF, GLU, false);
  }
  TW_REQUIRE(!GLU || N % 32 == 0);
  const int vec = N % 4 == 0 && (partial == nullptr || (uintptr_t)partial % 16 == 0) ? 1 : 0;
  auto kernel = gemm_stream_cu_kernel<T, OutT, MT, PARTIAL, GLU>;
  static bool attribute_set = false;   // per instantiation
  if (!attribute_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, TW_CU_LDS_BYTES);
    if (e != hipSuccess) return (int)e;
    attribute_set = true;
  }
  const int threads = TW_CU_WAVES * 64;
  kernel<<<plan.splits * plan.wgs_per_split, threads, TW_CU_LDS_BYTES, stream>>>(
      A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, M, N, K, plan.splits, plan.wgs_per_split, plan.compute_waves,
      plan.steps_per_split, vec);
  int err = TW_LAUNCH_RESULT();
  if (err || plan.splits == 1 || PARTIAL) return err;
  return launch_splitk_reduce<OutT>(partial, plan.splits, bias, residual, ldr, C, ldc, M, N, stream);
}

template <typename T, typename OutT, bool PARTIAL, bool GLU>
static int launch_stream_cu(const T* A, long lda, const T* W, long ldw, const float* bias, const float* residual,
                            long ldr, OutT* C, long ldc, float* partial, long partial_bytes, int M, int N, int K,
                            hipStream_t stream) {
  if (M <= 16) return launch_stream_cu_mt<T, OutT, 1, PARTIAL, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  if (M <= 32) return launch_stream_cu_mt<T, OutT, 2, PARTIAL, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  if (M <= 48) return launch_stream_cu_mt<T, OutT, 3, PARTIAL, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  return launch_stream_cu_mt<T, OutT, 4, PARTIAL, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
}

// Above this many rows (and up to 64) the kernel with one workgroup per CU runs for shuffled weights.
#define TW_CU_ABOVE_ROWS 16

template <typename T, typename OutT, bool PARTIAL, bool SHUF, bool GLU>
static int launch_skinny_lds_m(const T* A, long lda, const T* W, long ldw, const float* bias,
                               const float* residual, long ldr, OutT* C, long ldc, float* partial,
                               long partial_bytes, int M, int N, int K, hipStream_t stream) {
  if (M <= 16) return launch_skinny_lds<T, OutT, 1, PARTIAL, SHUF, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  if (M <= 32) return launch_skinny_lds<T, OutT, 2, PARTIAL, SHUF, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  if (M <= 48) return launch_skinny_lds<T, OutT, 3, PARTIAL, SHUF, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  return launch_skinny_lds<T, OutT, 4, PARTIAL, SHUF, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
}

// force: 0 = choose, 1 = generic, 3 = tiled 128x128, 4 = tiled 128x256, 5 = skinny, 6 = tiled 256x256,
// 7 = tiled 256x192, 8 = streaming with one workgroup per CU (shuffled weights, up to 64 rows)
template <typename T, typename OutT, bool SHUF, bool GLU>
static int linear_dispatch(const T* A, long lda, const T* W, long ldw, const float* bias,
                           const float* residual, long ldr, OutT* C, long ldc, float* partial,
                           long partial_bytes, int M, int N, int K, int force, hipStream_t stream) {
  constexpr int EPF = Elem<T>::kPerFrag;
  TW_REQUIRE(force == 0 || force == 1 || (force >= 3 && force <= 8));
  // the shuffled layout exists only for K that is a multiple of 16 bytes and is always aligned
  const bool aligned = K % EPF == 0 && lda % EPF == 0 && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0) &&
                       (SHUF || ldw % EPF == 0);
  if (force == 1 || !aligned) {
    TW_REQUIRE(force <= 1);
    TW_REQUIRE(!SHUF || K % EPF == 0);
    const long outputs = (long)M * (GLU ? N / 2 : N);
    gemm_generic_kernel<T, OutT><<<tw_div_up(outputs, 256), 256, 0, stream>>>(A, lda, W, ldw, bias, residual, ldr, C,
                                                                            ldc, M, N, K, SHUF ? 1 : 0, GLU ? 1 : 0);
    return TW_LAUNCH_RESULT();
  }
  if (force == 8 || (force == 0 && SHUF && M > TW_CU_ABOVE_ROWS && M <= 64)) {
    TW_REQUIRE(M <= 64 && SHUF);
    if constexpr (SHUF)
      return launch_stream_cu<T, OutT, false, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  }
  if (force == 5 || (force == 0 && M <= 64)) {
    TW_REQUIRE(M <= 64);
    return launch_skinny_lds_m<T, OutT, false, SHUF, GLU>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, stream);
  }
  const int shape = force == 3 ? 1 : (force == 4 ? 2 : (force == 6 ? 3 : (force == 7 ? 4 : 0)));
  return tw_tiled_linear(sizeof(T) == 4 ? TW_DTYPE_F32 : TW_DTYPE_BF16, sizeof(OutT) == 4 ? 1 : 0, SHUF ? 1 : 0,
                         GLU ? 1 : 0, shape, A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes,
                         M, N, K, stream);
}

template <typename T, typename OutT>
static int linear_layout(int shuffled, const T* A, long lda, const T* W, long ldw, const float* bias,
                         const float* residual, long ldr, OutT* C, long ldc, float* partial,
                         long partial_bytes, int M, int N, int K, int force, hipStream_t stream) {
  if (shuffled)
    return linear_dispatch<T, OutT, true, false>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, force, stream);
  return linear_dispatch<T, OutT, false, false>(A, lda, W, ldw, bias, residual, ldr, C, ldc, partial, partial_bytes, M, N, K, force, stream);
}

static bool weight_layout_ok(int dtype, int shuffled, long ldw, int K) {
  const int epf = dtype == TW_DTYPE_F32 ? 4 : 8;
  return shuffled ? (K % epf == 0 && ldw >= (K / epf + 3) / 4) : ldw >= K;
}

// C = A W^T (+bias) (+residual). out_f32 != 0: C is float32 whatever the input type (residual
// stream, logits); else C has the input type. `residual` may be C itself. `partial` is scratch
// for split-K (tw_linear_workspace_bytes). shuffled != 0: W is in the shuffled layout and ldw
// is the number of k-steps between its row blocks, at least ceil(K / (4 * elements per 16 bytes)).
extern "C" int tw_linear(int dtype, int out_f32, const void* A, long lda, const void* W, long ldw, int shuffled,
                         const float* bias, const float* residual, long ldr, void* C, long ldc,
                         float* partial, long partial_bytes, int M, int N, int K, int force,
                         hipStream_t stream) {
  TW_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K && ldc >= N);
  TW_REQUIRE(weight_layout_ok(dtype, shuffled, ldw, K));
  TW_REQUIRE(residual == nullptr || (ldr >= N && out_f32));
  if (M == 0) return 0;
  if (dtype == TW_DTYPE_F32)
    return linear_layout<float, float>(shuffled, (const float*)A, lda, (const float*)W, ldw, bias, residual, ldr,
                                       (float*)C, ldc, partial, partial_bytes, M, N, K, force, stream);
  if (dtype == TW_DTYPE_BF16) {
    if (out_f32)
      return linear_layout<bf16_t, float>(shuffled, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, bias, residual, ldr,
                                          (float*)C, ldc, partial, partial_bytes, M, N, K, force, stream);
    return linear_layout<bf16_t, bf16_t>(shuffled, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, bias, residual, ldr,
                                         (bf16_t*)C, ldc, partial, partial_bytes, M, N, K, force, stream);
  }
  return TW_ERR_BAD_ARGUMENT;
}

template <typename T>
static int glu_layout(int shuffled, const T* A, long lda, const T* W, long ldw, const float* bias, T* C, long ldc,
                      int M, int N, int K, int force, hipStream_t stream) {
  if (shuffled)
    return linear_dispatch<T, T, true, true>(A, lda, W, ldw, bias, nullptr, 0, C, ldc, nullptr, 0, M, N, K, force, stream);
  return linear_dispatch<T, T, false, true>(A, lda, W, ldw, bias, nullptr, 0, C, ldc, nullptr, 0, M, N, K, force, stream);
}

// Gated linear unit: W [N, K] holds gate and up rows interleaved in blocks of 16 (N a multiple
// of 32); C [M, N / 2] = silu(gate) * up in the input type. bias (may be null) is indexed like W's rows.
extern "C" int tw_linear_glu(int dtype, const void* A, long lda, const void* W, long ldw, int shuffled,
                             const float* bias, void* C, long ldc, int M, int N, int K, int force,
                             hipStream_t stream) {
  TW_REQUIRE(M >= 0 && N > 0 && N % 32 == 0 && K > 0 && lda >= K && ldc >= N / 2);
  TW_REQUIRE(weight_layout_ok(dtype, shuffled, ldw, K));
  if (M == 0) return 0;
  if (dtype == TW_DTYPE_F32)
    return glu_layout<float>(shuffled, (const float*)A, lda, (const float*)W, ldw, bias, (float*)C, ldc, M, N, K, force, stream);
  if (dtype == TW_DTYPE_BF16)
    return glu_layout<bf16_t>(shuffled, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, bias, (bf16_t*)C, ldc, M, N, K, force, stream);
  return TW_ERR_BAD_ARGUMENT;
}

// ---- decode-path form: few rows, 16-byte aligned K ------------------------------------
// Number of K ranges tw_linear_partials uses for an [N, K] weight (0: shape not supported).
extern "C" int tw_linear_partial_splits(int dtype, int N, int K) {
  const int epf = dtype == TW_DTYPE_F32 ? 4 : 8;
  if (K % epf) return 0;
  return skinny_lds_splits(N, K, epf);
}

// The same for M rows whose stride is LDA elements: up to 64 rows the streaming kernel's ranges; above,
// those of the tiled kernels (0 where they would not split K: the product with its epilogue is then the
// better call). Which tiled kernel runs, and so how it splits, depends on the rows' stride too.
extern "C" int tw_linear_partial_splits_rows(int dtype, int shuffled, int M, int N, int K, long lda) {
  const int epf = dtype == TW_DTYPE_F32 ? 4 : 8;
  if (M <= 64 && shuffled && M > TW_CU_ABOVE_ROWS && K % epf == 0)
    return cu_plan(tw_div_up(M, 16), N, K, epf, false, true).splits;
  if (M <= 64) return tw_linear_partial_splits(dtype, N, K);
  if (K % epf || lda < K) return 0;
  const int splits = tw_tiled_partial_splits(dtype, shuffled, lda, M, N, K);
  return splits > 1 ? splits : 0;
}

template <typename T>
static int partials_layout(int shuffled, const T* A, long lda, const T* W, long ldw, float* partial,
                           long partial_bytes, int M, int N, int K, hipStream_t stream) {
  if (shuffled && M > TW_CU_ABOVE_ROWS)
    return launch_stream_cu<T, float, true, false>(A, lda, W, ldw, nullptr, nullptr, 0, (float*)nullptr, N, partial, partial_bytes, M, N, K, stream);
  if (shuffled)
    return launch_skinny_lds_m<T, float, true, true, false>(A, lda, W, ldw, nullptr, nullptr, 0, (float*)nullptr, N, partial, partial_bytes, M, N, K, stream);
  return launch_skinny_lds_m<T, float, true, false, false>(A, lda, W, ldw, nullptr, nullptr, 0, (float*)nullptr, N, partial, partial_bytes, M, N, K, stream);
}

// partial[split][M][N] (float32) = A[:, K range of split] W[:, same]^T for every split; the caller's
// next kernel adds the splits up (with bias, residual, norm or rotation as it needs). Up to 64 rows the
// streaming kernel runs, above that the tiled kernels.
extern "C" int tw_linear_partials(int dtype, const void* A, long lda, const void* W, long ldw, int shuffled,
                                  float* partial, long partial_bytes, int M, int N, int K, hipStream_t stream) {
  TW_REQUIRE(M >= 1 && N > 0 && K > 0 && lda >= K);
  const int epf = dtype == TW_DTYPE_F32 ? 4 : 8;
  TW_REQUIRE(K % epf == 0 && lda % epf == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0);
  TW_REQUIRE(weight_layout_ok(dtype, shuffled, ldw, K) && (shuffled || ldw % epf == 0));
  if (M > 64) {
    // the caller sized `partial` for the ranges tw_linear_partial_splits_rows named: they must be the ones used
    const int expect = tw_tiled_partial_splits(dtype, shuffled, lda, M, N, K);
    TW_REQUIRE(expect >= 1 && partial_bytes == (long)expect * M * N * 4);
    int used = 0;
    const int err = tw_tiled_partials(dtype, shuffled, A, lda, W, ldw, partial, partial_bytes, M, N, K, &used, stream);
    if (err) return err;
    return used == expect ? 0 : TW_ERR_BAD_ARGUMENT;
  }
  if (dtype == TW_DTYPE_F32)
    return partials_layout<float>(shuffled, (const float*)A, lda, (const float*)W, ldw, partial, partial_bytes, M, N, K, stream);
  if (dtype == TW_DTYPE_BF16)
    return partials_layout<bf16_t>(shuffled, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, partial, partial_bytes, M, N, K, stream);
  return TW_ERR_BAD_ARGUMENT;
}
