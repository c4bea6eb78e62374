// The block-scaled GEMM for few rows (M <= 64): out[M,N] = (A 2^sfa)(B 2^sfb)^T with e4m3 or e2m1 operands.
//
// Such a problem is one pass over B, and a tile with a 128- or 256-row A panel would idle most of its
// MFMAs and leave the chip to a handful of workgroups.  Here a workgroup of 8 waves owns a group of
// 16 NT rows of B (= output columns) at a time and every row of A; its waves share K between them in
// turns of UP panel steps of 128 bytes, so the workgroup as a whole walks 16 NT whole rows of B.
//
// B goes straight from memory into the registers the MFMA takes: a lane's part of an operand is two
// 16-byte pieces of one row, 64 bytes apart, and the four lanes that share a row read 64 contiguous bytes
// of it per load instruction.  B's E8M0 bytes: a batch needs one scale word (the four K-blocks of a step)
// per row, step and tile; one load instruction fetches four of those words, one per group of 16 lanes, and
// a lane permute hands each lane the word of its row, of which it takes its K-block's byte (a byte load
// per lane and word, four times as many load instructions, cost 1.0-1.6 us of a launch at 8192 x 8192:
// measured by leaving them out; this way 16 x 8192 x 8192 e4m3 takes 16.6 against 16.85 us with B from
// memory and 12.9 against 13.6 us with B in the memory-side cache, e2m1 9.85 against 10.2 and 7.65 against 8.7).
//
// A comes out of the L2 (every workgroup reads all of A: M x K bytes, a few hundred KiB), and how it is
// asked for matters more than B's stream: loaded the way B is, every load instruction asks the L2 for 16
// half lines, and a launch of 64 rows spends half its time on them (measured by leaving A's loads out).
// So a wave moves the rows of A it is about to use into a region of LDS of its own with
// global_load_lds_dwordx4 -- 8 rows x 128 bytes, whole lines, per instruction, no registers -- and reads
// its fragments from there (16-byte chunks XOR-swizzled inside each group of 8 rows: conflict-free),
// and A's blocked scale chunks travel the same way.  No other wave reads that region: no barrier.
//
// A batch (UP steps) is in registers / LDS while the next one's loads are in flight.  All of a batch's
// memory instructions are written as assembly and counted by hand (one s_waitcnt per batch): the
// compiler does not see the LDS-DMA loads, and its own counts would make a batch wait for part of the
// next one.  The waves' partial sums meet in LDS and are added in wave order; one wave per 16 x 16
// output tile writes it.  K-blocks past the end of K (K % 128 != 0) enter with a scale of 2^-127 on both
// sides, which leaves the sums as they are; their payload bytes are valid bytes of the same row read again.
//
// The grid is persistent: a workgroup takes the column groups b, b + grid, ... and the batch it loads
// ahead may belong to its next group, so those loads are in flight under the reduction and the stores of
// the group in hand.
#include "mx_few_rows.hpp"

#include <atomic>

#include "dt_device.hpp"
#include "dt_host.hpp"

namespace dt {

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kFewWaves = 8;

// 16 bytes / one byte per lane at a base that is the same for the whole wave plus a 32-bit lane offset.
// The value arrives later: nothing may look at it before wait_loads.
__device__ __forceinline__ v4i load16_async(uint32_t lane_off, const uint8_t* wave_base) {
  v4i r;
  // (no streaming hint: the two pieces of a lane are the two halves of one line, and with the hint the
  // second asks memory again: 16 x 8192 x 8192 e4m3 17.6 against 16.4 us)
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(r) : "v"(lane_off), "s"(wave_base) : "memory");
  return r;
}
__device__ __forceinline__ int load_word_async(uint32_t lane_off, const uint8_t* wave_base) {
  int r;
  asm volatile("global_load_dword %0, %1, %2" : "=v"(r) : "v"(lane_off), "s"(wave_base) : "memory");
  return r;
}
// 16 bytes per lane from memory into LDS at lds_addr + 16 * lane, without a register in between
__device__ __forceinline__ void load16_to_lds_async(uint32_t lds_addr, uint32_t lane_off, const uint8_t* wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(lane_off), "s"(wave_base) : "memory");
}
// until at most N of this wave's loads are outstanding (they complete in the order they were issued)
template <int N>
__device__ __forceinline__ void wait_loads() {
  static_assert(N >= 0 && N < 64, "the counter has 6 bits");
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// MH: A's rows in halves of a 16-row tile (8 rows, one LDS-DMA instruction per step); the second half of
// the last tile is not fetched when no row of A lies in it (its sums are never stored)
template <bool FP4, int MH, int NT, int UP>
__global__ __launch_bounds__(kFewWaves* kWave) void mx_few_rows_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                                                                     const uint8_t* __restrict__ sfa, const uint8_t* __restrict__ sfb,
                                                                     int M, int N, int K, int64_t lda, int64_t ldb,
                                                                     uint16_t* __restrict__ out, int64_t ldo, int groups, int stagger) {
  constexpr int WAVES = kFewWaves;
  constexpr int MT = (MH + 1) / 2;
  constexpr int KC = FP4 ? 2 : 1;  // MFMAs, and blocked scale chunks, per panel step of 128 bytes of a row
  static_assert(MH >= 1 && MH <= 8 && NT >= 1 && NT <= 2 && UP >= 1, "at most 64 rows of A, 32 columns per group");
  // LDS of a wave: two sets of [A rows of a batch: step, tile, half of 8 rows, 8 rows x 128 B][A scale chunks of the batch]
  constexpr int kPanel = UP * MT * 2048;
  constexpr int kScaleLoads = (UP * KC + 1) / 2;  // of 1 KiB = two scale chunks
  constexpr int kSetBytes = kPanel + kScaleLoads * 1024, kWaveBytes = 2 * kSetBytes;
  static_assert(MT * NT * 1024 <= kPanel, "a wave parks its sums in the set it has just used up");
  // B's scale words of a batch: one per (step, chunk of the step, 16-column tile), number (u * KC + c) * NT + j.
  // One load instruction fetches four of them, one per group of 16 lanes (lane group g' of instruction i
  // has word 4 i + g' for the 16 rows of that tile), and the lanes that need a word take it from there with
  // a lane permute: a fourth of the load instructions that a byte per lane and word would be.
  constexpr int kBWords = UP * KC * NT, kBWordLoads = (kBWords + 3) / 4;
  // loads of a batch, in the order they are issued
  constexpr int kLoadsPerBatch = UP * NT * 2 + kBWordLoads + UP * MH + kScaleLoads;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x / kWave);
  const int l16 = lane & 15, g = lane >> 4;
  const uint32_t lds_wave = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds + (uint32_t)wave * kWaveBytes;
  uint8_t* const my_lds = lds + wave * kWaveBytes;
  const int k_bytes = FP4 ? K / 2 : K;                 // of a row
  const int p_steps = (k_bytes + 127) / 128;           // panel steps
  const int k_chunks = (K + 127) / 128;                // blocked scale chunks per 128 rows
  const int tail_p = (k_bytes % 128) ? p_steps - 1 : -1;  // a partly filled last step
  const int tail_chunks = (k_bytes % 128) / 16;

  // ---- per-lane offsets.  A, as LDS-DMA: lane L fills row L / 8, chunk position L % 8 of a group of 8
  // rows, i.e. it fetches logical chunk (L % 8) ^ (L / 8) of that row; in a partly filled step a chunk
  // past the end reads chunk c % (valid chunks) again (never the next row, never past the tensor).
  const int drow = lane >> 3, dchunk = (lane & 7) ^ drow;
  const uint32_t a_tail_adj = tail_chunks > 0 ? (uint32_t)(dchunk - dchunk % tail_chunks) * 16u : 0u;
  uint32_t oa[MT][2];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = t * 16 + h * 8 + drow;
      oa[t][h] = (uint32_t)(r < M ? r : M - 1) * (uint32_t)lda + dchunk * 16;
    }
  // A's fragments in LDS: row l16 of a tile = group l16 / 8, row l16 % 8; logical chunks g and 4 + g
  const uint32_t frag_lo = (l16 >> 3) * 1024 + (l16 & 7) * 128 + ((g ^ (l16 & 7)) << 4), frag_hi = frag_lo ^ 64u;
  // a row's scale word inside a 512-byte chunk of 128 rows; the lane's own byte is K-block g
  auto scale_word_offset = [&](int row) { return (uint32_t)((row & 31) * 16 + ((row & 127) >> 5) * 4); };
  auto scale_offset = [&](int row) { return scale_word_offset(row) + (uint32_t)g; };
  // which of B's scale words this lane fetches with load instruction i (clamped to the last one: fetched twice, used once)
  int bw_u[kBWordLoads], bw_c[kBWordLoads], bw_j[kBWordLoads];
#pragma unroll
  for (int i = 0; i < kBWordLoads; ++i) {
    const int n = 4 * i + g < kBWords ? 4 * i + g : kBWords - 1;
    bw_j[i] = n % NT;
    bw_c[i] = (n / NT) % KC;
    bw_u[i] = n / (NT * KC);
  }
  uint32_t osa[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) osa[t] = scale_offset(t * 16 + l16 < M ? t * 16 + l16 : M - 1);
  // B: the two pieces of a lane (bytes 16 g and 64 + 16 g of the step); in a partly filled step a piece
  // past the end reads the row's first piece of the step again
  const bool lo_in_tail = g < tail_chunks, hi_in_tail = 4 + g < tail_chunks;
  // what of B depends on the column group
  struct Group {
    const uint8_t *b0, *sb0;
    uint32_t ob[NT], osb[kBWordLoads];  // osb: the lane's scale word of load i inside its chunk
  };
  // Which group of columns a workgroup takes in a round of the grid.  Neighbouring groups share the 128-row
  // chunks of B's blocked scales (four groups of 32 columns per chunk), and workgroup b runs on XCD b % 8:
  // the groups 4 q .. 4 q + 3 go to four workgroups that follow one another on one XCD, so that its L2
  // fetches those lines once instead of four L2s fetching them once each (the counters read 8 % less
  // traffic per launch of 16 x 8192 x 8192).  `v` counts blockIdx.x, blockIdx.x + grid, ...
  const int wg = blockIdx.x, grid_size = gridDim.x;
  const int wg_spread = (grid_size % 32 == 0) ? ((wg >> 3) >> 2) * 32 + (wg & 7) * 4 + ((wg >> 3) & 3) : wg;
  auto columns_of = [&](int v) { return v - wg + grid_size <= groups ? v - wg + wg_spread : v; };
  auto group_at = [&](int v) {
    Group q;
    const int grp = columns_of(v);
    const int n0 = grp * (16 * NT);
    q.b0 = b + (int64_t)n0 * ldb;
    q.sb0 = sfb + (int64_t)(n0 >> 7) * k_chunks * 512;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int brow = n0 + j * 16 + l16 < N ? n0 + j * 16 + l16 : N - 1;  // rows past the edge re-read the last one; never stored
      q.ob[j] = (uint32_t)(brow - n0) * (uint32_t)ldb;
    }
#pragma unroll
    for (int i = 0; i < kBWordLoads; ++i) {
      const int brow = n0 + bw_j[i] * 16 + l16 < N ? n0 + bw_j[i] * 16 + l16 : N - 1;
      q.osb[i] = scale_word_offset(brow);
    }
    return q;
  };
  struct Batch {
    v4i blo[NT][UP], bhi[NT][UP];
    int sbw[kBWordLoads];
  };
  // Everything a batch needs is sent for here: kLoadsPerBatch instructions whatever the batch (a step
  // past the last one reads the last one again and counts as nothing, see consume)
  auto issue = [&](Batch& w, int set, const Group& q, int first_step) {
    const uint32_t lds_set = lds_wave + (uint32_t)set * kSetBytes;
#pragma unroll
    for (int u = 0; u < UP; ++u) {
      const int p = first_step + u < p_steps ? first_step + u : p_steps - 1;
      const bool tail = p == tail_p;
      const uint8_t* const bk = q.b0 + (int64_t)p * 128;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        w.blo[j][u] = load16_async(q.ob[j] + ((tail && !lo_in_tail) ? 0u : (uint32_t)g * 16u), bk);
        w.bhi[j][u] = load16_async(q.ob[j] + ((tail && !hi_in_tail) ? 0u : 64u + (uint32_t)g * 16u), bk);
      }
      const uint8_t* const ak = a + (int64_t)p * 128;
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          if (t * 2 + h < MH) load16_to_lds_async(lds_set + ((u * MT + t) * 2 + h) * 1024, oa[t][h] - (tail ? a_tail_adj : 0u), ak);
    }
#pragma unroll
    for (int i = 0; i < kBWordLoads; ++i) {  // (the chunk's offset is a lane's own here: below 4 K bytes, which the host has bounded)
      const int p = first_step + bw_u[i] < p_steps ? first_step + bw_u[i] : p_steps - 1;
      const int kc = p * KC + bw_c[i] < k_chunks ? p * KC + bw_c[i] : k_chunks - 1;
      w.sbw[i] = load_word_async((uint32_t)kc * 512u + q.osb[i], q.sb0);
    }
    // A's scale chunks of the batch are neighbours in the blocked buffer: 1 KiB = two chunks per instruction
    const int c0 = first_step * KC;
#pragma unroll
    for (int i = 0; i < kScaleLoads; ++i) {
      const int kc = c0 + 2 * i + (lane >> 5);
      load16_to_lds_async(lds_set + kPanel + i * 1024, (uint32_t)(kc < k_chunks ? kc : k_chunks - 1) * 512u + (lane & 31) * 16u, sfa);
    }
  };
  v4f acc[MT][NT];
  auto clear = [&]() {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};
  };
  // The batch has arrived (the caller has waited): MFMAs with A's fragments and scale bytes out of LDS
  auto consume = [&](Batch& w, int set, int first_step) {
    const uint8_t* const set_lds = my_lds + set * kSetBytes;
#pragma unroll
    for (int u = 0; u < UP; ++u) {
#pragma unroll
      for (int j = 0; j < NT; ++j) {  // from here on the loaded values may be looked at
        asm volatile("" : "+v"(w.blo[j][u]), "+v"(w.bhi[j][u]));
      }
      if (u == 0) {
#pragma unroll
        for (int i = 0; i < kBWordLoads; ++i) asm volatile("" : "+v"(w.sbw[i]));
      }
      // elements of K from this step on; the lane's K-block of MFMA c starts 128 c + 32 g elements in
      const int left = K - (first_step + u) * (FP4 ? 256 : 128);
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const bool valid = c * 128 + g * 32 < left;
        int sa[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) sa[t] = valid ? (int)set_lds[kPanel + (u * KC + c) * 512 + osa[t]] : 0;
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          // the tile's scale words sit in lane group n % 4 of load n / 4; this lane's K-block is byte g of its row's
          const int n = (u * KC + c) * NT + j;
          const int word = __builtin_amdgcn_ds_bpermute(((n % 4) * 16 + l16) * 4, w.sbw[n / 4]);
          const int sb = valid ? (int)__builtin_amdgcn_ubfe((uint32_t)word, (uint32_t)g * 8u, 8u) : 0;
          const v8i vb = FP4 ? __builtin_shufflevector(c == 0 ? w.blo[j][u] : w.bhi[j][u], v4i{0, 0, 0, 0}, 0, 1, 2, 3, 4, 5, 6, 7)
                             : __builtin_shufflevector(w.blo[j][u], w.bhi[j][u], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            const uint8_t* const f = set_lds + (u * MT + t) * 2048;
            const v4i alo = *reinterpret_cast<const v4i*>(f + frag_lo), ahi = *reinterpret_cast<const v4i*>(f + frag_hi);
            const v8i va = FP4 ? __builtin_shufflevector(c == 0 ? alo : ahi, v4i{0, 0, 0, 0}, 0, 1, 2, 3, 4, 5, 6, 7)
                               : __builtin_shufflevector(alo, ahi, 0, 1, 2, 3, 4, 5, 6, 7);
            // B as the row operand: acc[t][j][v] = D[row 16 t + l16][column n0 + 16 j + 4 g + v]
            acc[t][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb, va, acc[t][j], FP4 ? 4 : 0, FP4 ? 4 : 0, 0, sb, 0, sa[t]);
          }
        }
      }
    }
  };
  // The end of a group: every wave parks its sums in the set it has just used up (the other one may be
  // receiving the next batch), they are added in wave order (the same sum whatever the timing), and
  // wave t writes the output tiles t, t + 8, ...
  auto finish = [&](int v, int set) {
    const int grp = columns_of(v);
    v4f* const mine = reinterpret_cast<v4f*>(my_lds + set * kSetBytes);
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int j = 0; j < NT; ++j) mine[(t * NT + j) * kWave + lane] = acc[t][j];
    __syncthreads();
    const int n0 = grp * (16 * NT);
#pragma unroll
    for (int tile0 = 0; tile0 < MT * NT; tile0 += WAVES) {
      const int tile = tile0 + wave;
      if (tile < MT * NT) {
        v4f sum = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < WAVES; ++w) sum += reinterpret_cast<const v4f*>(lds + w * kWaveBytes + set * kSetBytes)[tile * kWave + lane];
        const int m = (tile / NT) * 16 + l16, n = n0 + (tile % NT) * 16 + 4 * g;
        if (m < M && n < N)  // N % 4 == 0: four columns or none
          *reinterpret_cast<u32x2*>(out + (int64_t)m * ldo + n) = u32x2{pack_bf16x2(sum.x, sum.y), pack_bf16x2(sum.z, sum.w)};
      }
    }
    __syncthreads();  // before anybody's next batch lands in that set
  };

  // A wave's batches of a group: wave, wave + 8, ... of UP steps each, the same number for every wave
  // (one past the last batch is sent for like any other and counts as nothing).  The workgroups do
  // not all start at the front of their rows: group number grp begins `rot` batches in and wraps around,
  // so that at any moment the chip's loads are spread over the whole length of the rows.
  const int batches = (p_steps + UP - 1) / UP, per_wave = (batches + WAVES - 1) / WAVES;
  auto first_step_of = [&](int grp, int i) {
    const int bi = wave + i * WAVES;
    if (bi >= batches) return p_steps;
    const int r = bi + (stagger ? (int)(((unsigned)grp * 5u) % (unsigned)batches) : 0);
    return (r >= batches ? r - batches : r) * UP;
  };
  // The sequence of (group, batch) pairs of this wave over two sets of registers and LDS: the pair after
  // the one being computed is already on its way, also across the end of a group.
  int grp = blockIdx.x, i = 0;
  if (grp >= groups) return;  // (the whole workgroup)
  auto advance = [&](int& gq, int& iq) {  // the pair after (gq, iq); gq >= groups: none
    if (++iq == per_wave) { iq = 0; gq += gridDim.x; }
  };
  Batch wa, wb;
  Group q = group_at(grp);
  int step = first_step_of(grp, i);
  issue(wa, 0, q, step);
  clear();
  for (;;) {
    // ---- set 0 holds (grp, i): send for its successor into set 1, then compute set 0
    int g2 = grp, i2 = i;
    advance(g2, i2);
    Group q2 = q;
    int step2 = 0;
    if (g2 < groups) {
      if (g2 != grp) q2 = group_at(g2);
      step2 = first_step_of(g2, i2);
      issue(wb, 1, q2, step2);
      wait_loads<kLoadsPerBatch>();
    } else {
      wait_loads<0>();
    }
    consume(wa, 0, step);
    if (g2 != grp) { finish(grp, 0); clear(); }
    if (g2 >= groups) break;
    grp = g2; i = i2; q = q2; step = step2;
    // ---- set 1 holds (grp, i): the same with the roles of the sets swapped
    advance(g2, i2);
    if (g2 < groups) {
      if (g2 != grp) q2 = group_at(g2);
      step2 = first_step_of(g2, i2);
      issue(wa, 0, q2, step2);
      wait_loads<kLoadsPerBatch>();
    } else {
      wait_loads<0>();
    }
    consume(wb, 1, step);
    if (g2 != grp) { finish(grp, 1); clear(); }
    if (g2 >= groups) break;
    grp = g2; i = i2; q = q2; step = step2;
  }
}

// Shape of the launch for a problem: 16-column tiles per group (NT), panel steps per batch (UP)
struct Plan {
  int nt, up;
};

constexpr size_t few_rows_lds_bytes(bool fp4, int mt, int up) {
  return (size_t)kFewWaves * 2 * ((size_t)up * mt * 2048 + (size_t)((up * (fp4 ? 2 : 1) + 1) / 2) * 1024);
}
constexpr size_t kLdsLimit = 160 * 1024;

// Two tiles per group halve the workgroups' reads of A (every group reads all of it) and win wherever they
// still give every CU a group (8192 x 8192, us, one tile / two: e4m3 1 row 16.2 / 15.6, 8 rows 16.8 / 15.8,
// 16 rows 18.3 / 16.5, 56 rows 28.9 / 20.9; e2m1 1 row 10.9 / 9.4, 56 rows 16.5 / 12.2).
Plan plan_for(bool fp4, int64_t M, int64_t N) {
  Plan p;
  const int tiles = tuning("gemm.few_rows_tiles");
  p.nt = tiles ? (tiles == 2 ? 2 : 1) : (N >= 32 * (int64_t)device_facts().cu_count ? 2 : 1);
  const int mt = (int)((M + 15) / 16);
  int up = tuning("gemm.few_rows_steps");
  if (up != 1 && up != 2) up = mt == 1 ? 2 : 1;
  if (up == 2 && (mt > 2 || few_rows_lds_bytes(fp4, mt, 2) >= kLdsLimit)) up = 1;
  p.up = up;
  return p;
}

template <bool FP4, int MH, int NT, int UP>
int launch_instance(const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M, int64_t N, int64_t K,
                    int64_t lda, int64_t ldb, uint16_t* out, int64_t ldo, int64_t groups, int64_t grid, int stagger,
                    hipStream_t stream) {
  constexpr size_t kLds = few_rows_lds_bytes(FP4, (MH + 1) / 2, UP);
  static_assert(kLds <= kLdsLimit, "two sets per wave fit the CU's LDS");
  auto kernel = mx_few_rows_kernel<FP4, MH, NT, UP>;
  if (kLds > 64 * 1024) {  // once per instantiation and device
    static std::atomic<bool> allowed[16];
    int dev = 0;
    (void)hipGetDevice(&dev);
    const bool tracked = dev >= 0 && dev < 16;
    if (!tracked || !allowed[dev].load(std::memory_order_relaxed)) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds) != hipSuccess) {
        (void)hipGetLastError();  // reported here; the next HIP call must not see it again
        return DT_ERR_LAUNCH;
      }
      if (tracked) allowed[dev].store(true, std::memory_order_relaxed);
    }
  }
  kernel<<<(unsigned)grid, kFewWaves * kWave, kLds, stream>>>(a, b, sfa, sfb, (int)M, (int)N, (int)K, lda, ldb, out, ldo, (int)groups,
                                                            stagger);
  return launch_status();
}

}  // namespace

// What the kernel takes at all: its 32-bit lane offsets into A's blocked scales span 4 K bytes
bool few_rows_fits(int64_t M, int64_t K) { return M <= 64 && K <= ((int64_t)1 << 29); }

// Where the kernel above beats the 128 x 128 tiles that share K through a workspace (measured on MI355X,
// us, B rotated through enough buffers that it comes from HBM; few rows / tiles):
//   8192 x 8192:  e4m3 M = 8 15.7 / 20.7, 16 16.4 / 20.0, 32 18.1 / 20.5, 64 21.7 / 21.8; e2m1 10.1 / 21.8, 10.5 / 21.9, 11.6 / 22.0, 13.0 / 22.3
//   4096 x 14336 (N x K): e4m3 16.5 / 20.8, 18.5 / 21.3, 22.0 / 21.6, 26.9 / 23.0; e2m1 9.9 / 18.1 ... 14.3 / 19.4
//   16384 x 4096: e4m3 15.3 / 20.3, 16.0 / 20.3, 18.9 / 20.6, 23.9 / 22.0; e2m1 11.1 / 14.4 ... 14.1 / 14.3
//   2048 x 8192, 1024 x 8192, 4096 x 4096, 8192 x 2048: 0.25 to 0.7 of the tiles' time for every M
//   28672 x 4096: e4m3 27.2 / 31.1, 28.7 / 28.9, 33.3 / 29.1, 41.4 / 30.3; e2m1 17.4 / 16.5 ... 24.3 / 16.8
//   32768 x 1024: 1.1 to 1.9 times the tiles' time
// A group of columns costs its reduction and two barriers whatever K is, so many groups with a short K
// lose; and with e4m3 operands and more than 32 rows the workgroups' reads of A (every workgroup reads
// all of it) weigh as much as B once the problem is large.
bool few_rows_pays(bool fp4, int64_t M, int64_t N, int64_t K, bool have_workspace) {
  (void)have_workspace;
  if (!few_rows_fits(M, K)) return false;
  if (N < 1024 || K < 2048) return false;
  if (K < 8192 && N > 16384) return false;
  if (!fp4 && M > 32 && N * K > ((int64_t)1 << 25)) return false;
  return true;
}

int launch_few_rows(bool fp4, const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M, int64_t N,
                    int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo, hipStream_t stream) {
  uint16_t* o = static_cast<uint16_t*>(out);
  const Plan p = plan_for(fp4, M, N);
  const int mh = (int)((M + 7) / 8);  // halves of 16-row tiles that hold rows of A
  const int64_t groups = ceil_div(N, (int64_t)16 * p.nt);
  int per_cu = tuning("gemm.few_rows_per_cu");
  if (per_cu < 1) per_cu = 2;
  int64_t grid = groups;
  if (grid > (int64_t)device_facts().cu_count * per_cu) grid = (int64_t)device_facts().cu_count * per_cu;
  const int stagger = tuning("gemm.few_rows_stagger");
#define DT_FEW(FP4, MH, NT, UP) return launch_instance<FP4, MH, NT, UP>(a, b, sfa, sfb, M, N, K, lda, ldb, o, ldo, groups, grid, stagger, stream)
#define DT_FEW_U(FP4, MH, NT)                                                      \
  do {                                                                             \
    if constexpr (MH <= 4 && few_rows_lds_bytes(FP4, (MH + 1) / 2, 2) < kLdsLimit) { if (p.up == 2) DT_FEW(FP4, MH, NT, 2); } \
    DT_FEW(FP4, MH, NT, 1);                                                        \
  } while (0)
#define DT_FEW_N(FP4, MH) do { if (p.nt == 2) DT_FEW_U(FP4, MH, 2); else DT_FEW_U(FP4, MH, 1); } while (0)
#define DT_FEW_M(FP4)                         \
  do {                                        \
    switch (mh) {                             \
      case 1: DT_FEW_N(FP4, 1);               \
      case 2: DT_FEW_N(FP4, 2);               \
      case 3: DT_FEW_N(FP4, 3);               \
      case 4: DT_FEW_N(FP4, 4);               \
      case 5: DT_FEW_N(FP4, 5);               \
      case 6: DT_FEW_N(FP4, 6);               \
      case 7: DT_FEW_N(FP4, 7);               \
      default: DT_FEW_N(FP4, 8);              \
    }                                         \
  } while (0)
  if (fp4) DT_FEW_M(true);
  else DT_FEW_M(false);
#undef DT_FEW_M
#undef DT_FEW_N
#undef DT_FEW_U
#undef DT_FEW
  return DT_ERR_LAUNCH;  // not reached
}

}  // namespace dt
