// The block-scaled GEMM on the CDNA4 scaled MFMA: kernel, launch plans and argument checks shared by
// dt_mx_fp8_bf16 (mx_fp8_bf16.hip) and dt_mx_fp4_bf16 (mx_fp4_bf16.hip), which are compiled separately.
//
// D[M,N] = sum_k (A[m,k] 2^(sfa[m,k/32]-127)) (B[n,k] 2^(sfb[n,k/32]-127)); A is [M,K] and B is
// [N,K], both with K contiguous.  Operand layout of v_mfma_scale_f32_16x16x128_f8f6f4 (measured
// on gfx950): lane l = 16*g + i supplies, for row i, K = 16g..16g+15 in its first four VGPRs
// and K = 64+16g..64+16g+15 in the last four; the E8M0 byte lane l supplies scales K-block g
// (K = 32g..32g+31) of row i.  So a fragment is two 16-byte reads 64 bytes apart, and one MX
// block maps to one scale lane.
//
// A workgroup of 4 waves owns a BM x BN output tile and walks K in steps of 128.  The A and B
// panels of a step go from global memory straight into LDS (global_load_lds_dwordx4: lane L of
// a wave deposits its 16 bytes at LDS base + 16 L, so one wave instruction fills 8 rows of
// 128 bytes) into a ring of NST stages, with one barrier per step placed in the middle of the
// step's MFMA stream (see the main loop).  Inside an 8-row group the 16-byte chunks of row
// r sit at chunk ^ (r & 7), which makes the 16-byte fragment reads of 16 consecutive rows
// conflict-free (measured: 6.25 clk per wave read, the same as a linear read; 144-byte padded
// rows cost 8, unswizzled rows 16).  The step's E8M0 scale chunks of the blocked buffers
// travel the same way; a 16-byte LDS read returns the scale words of four row tiles at once.
// The MFMA is issued with B as the row operand, so a lane's four accumulators are four
// consecutive columns of one output row; the epilogue converts to bf16 and goes through LDS so
// that the stores are whole 256-byte row segments (direct 8-byte stores cost 12% of the run).
#pragma once

#include <atomic>
#include <type_traits>

#include "dt_device.hpp"
#include "dt_host.hpp"
#include "mx_few_rows.hpp"

namespace dt {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kBK = 128;             // K bytes per step = one 16x16x128 MFMA
constexpr int kGroupRows = 8;        // rows filled by one wave-wide LDS-DMA load
constexpr int kGroupStride = 1024;   // 8 rows of 128 bytes; the chunk swizzle alone makes fragment reads conflict-free (measured)
constexpr size_t kSplitTicketBytes = 1024;        // head of the split-K workspace: one counter per 128 x 128 tile
constexpr size_t kSplitTileBytes = 128 * 128 * 4;  // parked fp32 accumulators of one tile and split
constexpr int kMaxSplits = 16;      // what gemm.split_k may force
constexpr int kAutoMaxSplits = 12;  // what the library picks by itself

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// FP4: both operands are e2m1 nibbles, two per byte with the even element in the low nibble
// (measured on gfx950: with format 4 lane 16g+i supplies row i, K = 32g..32g+31 in its first
// four VGPRs, element k in nibble k%8 of word (k%32)/8).  A 128-byte LDS row then holds 256
// elements = two MFMAs: bytes 16g.. of the first half feed the first, bytes 64+16g.. the second,
// which are the same two 16-byte reads a lane makes for e4m3.  Everything else (panels, DMA,
// swizzle, ring, quadrant schedule, epilogue) is shared; a K-step carries twice the scales.
//
// SPLIT: the K-steps of a tile are shared between `splits` workgroups (workgroup = tile + split *
// tiles).  Each parks its fp32 accumulators in `partial`, lane for lane, and takes a ticket of
// its tile; whoever draws the last ticket adds the parked accumulators in split order (so the sum
// does not depend on who came last), writes the bf16 tile and puts the ticket counter back to
// zero.  Nobody waits for anybody.
// The parked accumulators travel as device-scope relaxed atomics (stores that write through the
// XCD's L2, loads that miss it): ordinary stores would need a release and an acquire fence around
// the ticket, i.e. a write-back and an invalidation of the whole L2 that every other workgroup
// of the XCD is reading its panels through (measured: 1024^3 20.5 us with the fences, 8.8 us
// without splitting).
//
// MODE kQuads: the workgroup computes one 128 x 128 quadrant of a 256 x 256 tile, for the tiles that
// the 256 x 256 kernel leaves over when its grid is cut to whole rounds of the chip (tiles_m,
// tiles_n and first_block then describe the 256 x 256 tiling).
// MODE kHalves: the same with the 256 x 128 halves of a tile.
enum GemmMode { kPlain = 0, kSplitK = 1, kQuads = 2, kHalves = 3 };
// KTAIL: the last K-step is partly filled (K is not a multiple of 128 bytes of a row).  Everything that
// deals with it is compiled only then: a branch or two in the K loop cost the kernel for whole steps 3 to
// 6 % (measured), whatever they guard.
template <int BM, int BN, int WAVES_M, int WAVES_N, int NST, bool FP4, bool TOUCH, int MODE, bool KTAIL>
__global__ __launch_bounds__(WAVES_M* WAVES_N* kWave) void mx_gemm_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, const uint8_t* __restrict__ sfa,
    const uint8_t* __restrict__ sfb, int M, int N, int K, int64_t lda, int64_t ldb, uint16_t* __restrict__ out,
    int64_t ldo, int tiles_m, int tiles_n, int wide_stores, int splits, v4f* __restrict__ partial,
    uint32_t* __restrict__ tickets, int first_block, uint64_t* __restrict__ phase_log) {
  constexpr bool SPLIT = MODE == kSplitK;
  // phase_log (only in a build with DT_PHASE_LOG, and normally null there; dt_set_phase_log): per workgroup
  // four readings of the 100 MHz constant-rate counter -- start, K loop entered, K loop left, output
  // stored -- and where it ran (XCC_ID, HW_ID), stored at the very end.
  auto clock_reading = []() -> uint64_t {
    if constexpr (kPhaseLog) return wall_clock64();
    else return 0;
  };
  const uint64_t t_start = clock_reading();
  static_assert(!(SPLIT && TOUCH), "the prefetch shares assume that a workgroup walks the whole K");
  static_assert(MODE != kQuads || (BM == 128 && BN == 128), "quadrants of a 256 x 256 tile");
  static_assert(MODE != kHalves || (BM == 256 && BN == 128), "halves of a 256 x 256 tile");
  constexpr bool PARTS = MODE == kQuads || MODE == kHalves;
  constexpr int kParts = MODE == kQuads ? 4 : 2;  // workgroups per 256 x 256 tile
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // wave tile
  constexpr int TM = WM / 16, TN = WN / 16;            // MFMA tiles per wave
  constexpr int KC = FP4 ? 2 : 1;                      // 128-element MFMAs (and blocked scale chunks) per K-step

  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int kGroupsA = BM / kGroupRows, kGroupsB = BN / kGroupRows;
  constexpr int kPanelA = kGroupsA * kGroupStride, kPanelB = kGroupsB * kGroupStride;
  constexpr int kScaleA = 1024 * KC, kScaleB = 1024 * KC;  // per chunk of the K-step: two 512-byte blocked scale chunks (2 x 128 rows)
  constexpr int kOffB = kPanelA, kOffSA = kPanelA + kPanelB, kOffSB = kOffSA + kScaleA;
  constexpr int kStageBytes = kOffSB + kScaleB;  // one K-step: A panel, B panel, A scales, B scales
  constexpr int kWaves = WAVES_M * WAVES_N;
  constexpr int kLoadsA = kGroupsA / kWaves, kLoadsB = kGroupsB / kWaves;  // DMA loads per wave and step
  static_assert(kLoadsA * kWaves == kGroupsA && kLoadsB * kWaves == kGroupsB, "tile/waves mismatch");
  static_assert(BM % 128 == 0 && BN % 128 == 0 && BM <= 256 && BN <= 256, "scale chunks are 128 rows");

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // Workgroups are handed to the 8 XCDs round-robin; give each XCD a contiguous run of tile
  // ids so that neighbours in the tile grid share an L2, then walk tiles in column groups.
  int bid = blockIdx.x;
  const int nb = tiles_m * tiles_n;
  int split = 0, quad = 0;
  if constexpr (SPLIT) {
    split = bid / nb;
    bid -= split * nb;
  }
  if constexpr (PARTS) {
    // workgroup 8 * (kParts * g + part) + x: part `part` of tile first_block + 8 g + x, so that a tile's
    // parts run on one XCD (x) and first_block (a multiple of 8) continues the big kernel's runs
    const int t = bid >> 3;
    quad = t % kParts;
    bid = first_block + 8 * (t / kParts) + (bid & 7);
    if (bid >= nb) return;  // the grid is rounded up to whole groups of 8 tiles
  }
  if (nb % 8 == 0) bid = (bid % 8) * (nb / 8) + bid / 8;
  constexpr int kGroup = 8;  // tile rows per group
  const int group_size = kGroup * tiles_n;
  const int g = bid / group_size, first_m = g * kGroup;
  const int gm = (tiles_m - first_m) < kGroup ? (tiles_m - first_m) : kGroup;
  const int tile_m = first_m + (bid % group_size) % gm;
  const int tile_n = (bid % group_size) / gm;
  const int m0 = MODE == kQuads ? tile_m * 256 + (quad >> 1) * 128 : tile_m * BM;
  const int n0 = PARTS ? tile_n * 256 + (quad & 1) * 128 : tile_n * BN;
  if constexpr (PARTS) {
    if (m0 >= M || n0 >= N) return;  // quadrant outside the matrix (the whole workgroup leaves)
  }
  // K counts elements (a multiple of 32, the MX block); a row holds k_bytes bytes, a K-step is 128 of
  // them.  The last step may be partly filled.  Its loads then stay inside the row: a 16-byte chunk past
  // the end reads a valid chunk of the same row again (tail_adj), and what it reads does not count,
  // because the scale bytes of its K-blocks are zero: byte 0 on both sides scales the block's sum by
  // 2^-254, which leaves the accumulator as it is (the re-read payload is finite unless the row holds
  // a NaN, and then the row's results are NaN anyway).  Those bytes are the padding of the caller's
  // blocked scale buffers, which nobody can check: whatever they hold, the staged copy of the partly
  // filled step's scale chunks is overwritten with zeros there before anybody reads it
  // (mask_tail_scales).  With FP4 a step is two
  // 128-element scale chunks; when the last step has no second chunk at all (K % 256 in 1..128) its
  // second MFMA is switched off through the scale operand (see scale_bits).
  const int k_bytes = FP4 ? K / 2 : K;
  int k_steps = (k_bytes + kBK - 1) / kBK;
  const int k_chunks = (K + 127) / 128;                           // blocked scale chunks per 128 rows
  int tail_step = KTAIL ? k_steps - 1 : -1;                            // index of a partly filled step
  int half_step = (KTAIL && FP4 && (k_chunks & 1)) ? k_steps - 1 : -1;  // index of a step without a second scale chunk
  // SPLIT: this workgroup walks steps ks_begin .. ks_begin + k_steps; from here on steps and scale
  // chunks count from ks_begin (the host makes sure that every split owns a step)
  int ks_begin = 0, k_chunks_left = k_chunks;
  if constexpr (SPLIT) {
    const int per = (k_steps + splits - 1) / splits;
    ks_begin = split * per;
    k_steps = k_steps - ks_begin < per ? k_steps - ks_begin : per;
    half_step -= ks_begin;
    tail_step -= ks_begin;
    k_chunks_left -= ks_begin * KC;
  }

  // ---- global -> LDS.  Wave w owns groups w*kLoads .. of each panel; lane L fills row L/8,
  // chunk position L%8 of the group, i.e. it fetches logical chunk (L%8) ^ (L/8) of that row.
  // Rows past the edge re-read the last row; their products are never stored.  The tile's first
  // row goes into the 64-bit scalar base, so the 32-bit lane offsets only span the tile's rows
  // and an operand may be larger than 4 GiB.
  // The loads of a panel go out in runs of four: the instruction's immediate offset counts on both sides
  // (global address and LDS address), so M0 and its wait state are paid once per run and the other
  // three loads are one instruction each.  Load n of a run carries offset n * kGroupStride; its lane
  // offset is lowered by as much, and the scalar bases by kRunBias so that no lane offset goes negative.
  constexpr uint32_t kRun = 4, kRunBias = (kRun - 1) * kGroupStride;
  const uint8_t* const A_tile = A + (int64_t)m0 * lda + (int64_t)ks_begin * kBK - kRunBias;
  const uint8_t* const B_tile = B + (int64_t)n0 * ldb + (int64_t)ks_begin * kBK - kRunBias;
  const int lrow = lane >> 3, lchunk = (lane & 7) ^ lrow;
  // in a partly filled step of v valid chunks, chunk c >= v reads chunk c % v again
  const int tail_chunks = (k_bytes % kBK) / 16;
  const uint32_t tail_adj = tail_chunks > 0 ? (uint32_t)(lchunk - lchunk % tail_chunks) * 16u : 0u;
  uint32_t offA[kLoadsA], offB[kLoadsB];
#pragma unroll
  for (int i = 0; i < kLoadsA; ++i) {
    int gr = m0 + (wave * kLoadsA + i) * kGroupRows + lrow;
    gr = gr < M ? gr : M - 1;
    offA[i] = (uint32_t)((int64_t)(gr - m0) * lda + lchunk * 16) + kRunBias - (i % kRun) * kGroupStride;
  }
#pragma unroll
  for (int i = 0; i < kLoadsB; ++i) {
    int gr = n0 + (wave * kLoadsB + i) * kGroupRows + lrow;
    gr = gr < N ? gr : N - 1;
    offB[i] = (uint32_t)((int64_t)(gr - n0) * ldb + lchunk * 16) + kRunBias - (i % kRun) * kGroupStride;
  }
  // Scales: KC more wave-wide loads per step.  Even waves bring A chunks, odd waves B chunks:
  // lanes 0-31 the tile's first 128-row chunk, lanes 32-63 the next one (the second chunk of a
  // 256-row tile; for a 128-row tile it lands in an unused half of the slot).  Every wave issues
  // them (duplicates write identical bytes), which keeps the instruction stream free of branches.
  const bool wave_is_b = (wave & 1) != 0;
  const int chunk_max = (wave_is_b ? (N + 127) / 128 : (M + 127) / 128) - 1;
  const int chunk0 = (wave_is_b ? n0 : m0) / 128;  // the tile's first chunk row: part of the scalar base
  const int chunk = chunk0 + (lane >> 5) < chunk_max ? chunk0 + (lane >> 5) : chunk_max;
  const uint8_t* sc_base = (wave_is_b ? sfb : sfa) + ((int64_t)chunk0 * k_chunks + (int64_t)ks_begin * KC) * 512;
  const uint32_t sc_off = (uint32_t)((int64_t)(chunk - chunk0) * k_chunks * 512 + (lane & 31) * 16);
  const int sc_dst = wave_is_b ? kOffSB : kOffSA;
  // load number n of a step: n < kLoadsA -> A group, < kLoadsA+kLoadsB -> B group, else scales
  constexpr int kLoadsPerStep = kLoadsA + kLoadsB + KC;
  // global_load_lds_dwordx4 in its scalar-base + 32-bit-lane-offset form (the builtin is
  // selected with a 64-bit address per lane, which costs a 64-bit add and a second address
  // register per load); M0 carries the LDS destination of the run's first load.
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;
  static_assert(kRun == 4 && kGroupStride == 1024, "the immediate offsets below");
  auto dma16 = [&](int run_pos, const uint8_t* uniform_base, uint32_t lane_off, uint32_t lds_off) {
    // M0 has no other user in this kernel (LDS reads do not need it on gfx9+)
    if (run_pos == 0)
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :
                   : "s"(lds_base + lds_off), "v"(lane_off), "s"(uniform_base)
                   : "memory");
    else if (run_pos == 1)
      asm volatile("global_load_lds_dwordx4 %0, %1 offset:1024" : : "v"(lane_off), "s"(uniform_base) : "memory");
    else if (run_pos == 2)
      asm volatile("global_load_lds_dwordx4 %0, %1 offset:2048" : : "v"(lane_off), "s"(uniform_base) : "memory");
    else
      asm volatile("global_load_lds_dwordx4 %0, %1 offset:3072" : : "v"(lane_off), "s"(uniform_base) : "memory");
  };
  // adj: what a lane's offset gives way by in a partly filled step (the prologue passes it; in the K loop
  // the offsets themselves are lowered once, see tail_in_place, so that a refill is one instruction)
  // the scalar bases of a step's loads
  struct StepBases {
    const uint8_t *a, *b, *s[KC];
  };
  auto base_a = [&](int ks) { return A_tile + (int64_t)ks * kBK; };
  auto base_b = [&](int ks) { return B_tile + (int64_t)ks * kBK; };
  auto base_s = [&](int ks, int c) {  // chunk c of the step; past the end it re-reads the last one (switched off)
    int kc = ks * KC + c;
    kc = kc < k_chunks_left ? kc : k_chunks_left - 1;
    return sc_base + (int64_t)kc * 512;
  };
  auto fetch_one = [&](int n, const StepBases& at, uint32_t buf, uint32_t adj) {
    if (n < kLoadsA) {
      dma16(n % kRun, at.a, offA[n] - adj, buf + (wave * kLoadsA + n - n % kRun) * kGroupStride);
    } else if (n < kLoadsA + kLoadsB) {
      const int i = n - kLoadsA;
      dma16(i % kRun, at.b, offB[i] - adj, buf + kOffB + (wave * kLoadsB + i - i % kRun) * kGroupStride);
    } else {
      const int c = n - kLoadsA - kLoadsB;
      dma16(0, at.s[c], sc_off, buf + sc_dst + c * 1024);
    }
  };
  auto tail_in_place = [&]() {
    asm volatile("; partly filled last step: lane offsets lowered for good" ::: "memory");  // keeps this a branch
#pragma unroll
    for (int i = 0; i < kLoadsA; ++i) offA[i] -= tail_adj;
#pragma unroll
    for (int i = 0; i < kLoadsB; ++i) offB[i] -= tail_adj;
  };
  auto fetch = [&](int ks, uint32_t buf) {
    StepBases at;
    at.a = base_a(ks);
    at.b = base_b(ks);
#pragma unroll
    for (int c = 0; c < KC; ++c) at.s[c] = base_s(ks, c);
#pragma unroll
    for (int n = 0; n < kLoadsPerStep; ++n) fetch_one(n, at, buf, KTAIL && ks == tail_step ? tail_adj : 0u);
  };
  // L2 prefetch (TOUCH).  The refill of a stage is issued one K-step before it is needed, which
  // is shorter than an L2 miss; and every panel line is an L2 miss for the first workgroup of
  // the XCD that asks for it.  So each workgroup also "touches" lines of a K-step further ahead
  // with one 4-byte LDS-DMA load per wave (no register destination; the bytes land in a dump
  // area nobody reads).  The 4 tile columns that share an A panel inside an XCD (and the 8 tile
  // rows that share a B panel) split the panel's lines between them: 64 lines of A and 32 of B
  // per workgroup and step, 96 / waves per wave.  A line nobody touched is merely slower.
  constexpr int kTouch = TOUCH ? 1 : 0;       // touch loads per wave and step
  constexpr int kTouchAhead = 2;              // K-steps ahead of the stage refill
  constexpr int kVmPerStep = kLoadsPerStep + kTouch;
  const uint8_t* touch_ptr = A;
  if constexpr (TOUCH) {
    static_assert(BM == 256 && BN == 256 && 96 % kWaves == 0, "touch shares are laid out for the 256 x 256 tile");
    constexpr int kTouchLines = 96 / kWaves;  // per wave
    const int idx = wave * kTouchLines + (lane < kTouchLines ? lane : kTouchLines - 1);  // 0..95: 64 lines of A, then 32 of B
    if (idx < 64) {
      int r = m0 + (tile_n & 3) * 64 + idx;
      r = r < M ? r : M - 1;
      touch_ptr = A + (int64_t)r * lda;
    } else {
      int r = n0 + (tile_m & 7) * 32 + (idx - 64);
      r = r < N ? r : N - 1;
      touch_ptr = B + (int64_t)r * ldb;
    }
  }
  auto touch_address = [&](int step) -> const uint8_t* {
    const int kt = step < k_steps ? step : k_steps - 1;
    return touch_ptr + (uint32_t)kt * kBK;
  };
  auto touch_at = [&](const uint8_t* p) {
    if constexpr (TOUCH) {
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                   :
                   : "s"(lds_base + (uint32_t)(NST * kStageBytes)), "v"(p)
                   : "memory");
    }
  };
  auto touch = [&](int step) { touch_at(touch_address(step)); };

  // The staged scale chunks of the partly filled step, once they have landed in ring slot `stage`: a
  // word holds the four K-block bytes of a row; the bytes of K-blocks past the end of K become 0.  A
  // slot is 256 words per operand and chunk, one per thread; the caller puts a barrier behind this.
  static_assert(kWaves * kWave * 4 == 1024, "one scale word per thread and 1 KiB slot");
  const int k_blocks = K / 32;
  auto mask_tail_scales = [&](uint32_t stage) {
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int valid = k_blocks - ((ks_begin + tail_step) * KC + c) * 4;  // K-blocks of this chunk inside K
      if (valid >= 4) continue;
      const uint32_t keep = valid <= 0 ? 0u : (1u << (8 * valid)) - 1u;
      uint32_t* const wa = reinterpret_cast<uint32_t*>(lds + stage + kOffSA + c * 1024) + tid;
      uint32_t* const wb = reinterpret_cast<uint32_t*>(lds + stage + kOffSB + c * 1024) + tid;
      *wa &= keep;
      *wb &= keep;
    }
  };

  v4f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  // fragment of tile row `l16` of a 16-row tile starting at panel row `row0` (multiple of 16):
  // logical chunks kq and 4+kq of the row, which sit 64 bytes apart (xor 4).  e4m3: K = 16kq..
  // and 64+16kq.. of one MFMA; e2m1: K = 32kq.. of the step's first and of its second MFMA.
  struct Frag {
    v4i lo, hi;
  };
  const int kq = lane >> 4, l16 = lane & 15;
  const uint32_t frag_lo = (l16 >> 3) * kGroupStride + (l16 & 7) * 128 + ((kq ^ (l16 & 7)) << 4);
  const uint32_t frag_hi = frag_lo ^ 64u;  // stage and panel offsets are multiples of 1024: the xor commutes with them
  auto load_frag = [&](uint32_t stage_lo, uint32_t stage_hi, int panel_off, int row0) -> Frag {
    // stage_lo/hi = stage offset + frag_lo/hi (one add each per K-step); the rest is an immediate
    const int o = panel_off + (row0 >> 3) * kGroupStride;
    return Frag{*reinterpret_cast<const v4i*>(lds + stage_lo + o), *reinterpret_cast<const v4i*>(lds + stage_hi + o)};
  };
  // Scales of a staged 512-byte chunk (128 rows): the word of row r sits at
  // (r%32)*16 + (r/32)*4, so the 16 bytes at (r%32)*16 hold the words of rows r%32 + {0,32,64,96},
  // i.e. of the four 16-row tiles t with the same parity (even tiles at l16*16, odd tiles 256
  // bytes on).  A half of the wave tile (H tiles) is 8 or 4 bytes of each group.  A word holds
  // the 4 K-block bytes of a row; the lane's own (K-block lane/16) goes to byte 0.
  constexpr int HA = TM / 2, HB = TN / 2;  // tiles in a half of the wave tile, per operand
  struct HalfWords {
    uint32_t w[KC][4];  // [chunk of the step][tile of the half]
  };
  // BYTES (e4m3, and only for scales that are used in the basic block that loads them, i.e. in the step
  // they belong to): each lane reads the one byte it needs, the K-block lane / 16 of its row's word, and
  // nothing has to be shifted.  Across the loop's back edge the compiler would move the byte's zero
  // extension to the other side, between the last MFMA of one step and the first of the next.
  auto read_half_scales = [&](auto h_tag, uint32_t o, int half, auto bytes_tag) -> HalfWords {  // o: stage + operand slot + lane part
    constexpr int H = decltype(h_tag)::value;
    constexpr bool BYTES = decltype(bytes_tag)::value && !FP4;
    if constexpr (BYTES) o += kq;
    HalfWords r;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      if constexpr (BYTES) {
        if constexpr (H == 4) {
          r.w[c][0] = lds[o + c * 1024 + half * 8];       r.w[c][1] = lds[o + c * 1024 + 256 + half * 8];
          r.w[c][2] = lds[o + c * 1024 + half * 8 + 4];   r.w[c][3] = lds[o + c * 1024 + 256 + half * 8 + 4];
        } else {
          r.w[c][0] = lds[o + c * 1024 + half * 4];
          r.w[c][1] = lds[o + c * 1024 + 256 + half * 4];
        }
      } else if constexpr (H == 4) {
        const u32x2 e = *reinterpret_cast<const u32x2*>(lds + o + c * 1024 + half * 8);
        const u32x2 d = *reinterpret_cast<const u32x2*>(lds + o + c * 1024 + 256 + half * 8);
        r.w[c][0] = e.x; r.w[c][1] = d.x; r.w[c][2] = e.y; r.w[c][3] = d.y;
      } else {
        r.w[c][0] = *reinterpret_cast<const uint32_t*>(lds + o + c * 1024 + half * 4);
        r.w[c][1] = *reinterpret_cast<const uint32_t*>(lds + o + c * 1024 + 256 + half * 4);
      }
    }
    return r;
  };
  // The scale operand: the lane's byte moved to bits 0-7.  For the second chunk of a half-filled
  // step the field width is 0, so the byte reads as 0 = 2^-127: the MFMA's sum is scaled by
  // 2^-254, underflows to zero (e2m1 has neither infinities nor NaNs) and leaves the accumulator
  // as it is.
  const uint32_t scale_shift = kq * 8;
  auto scale_bits = [&](uint32_t word, int c, int step) -> int {  // of a word
    if (KTAIL && FP4 && c == 1) return (int)__builtin_amdgcn_ubfe(word, scale_shift, step == half_step ? 0u : 8u);
    return (int)(word >> scale_shift);
  };
  // These scales are used on the other side of the loop's back edge, and left alone the compiler moves
  // their shifts over there, between the last MFMA of one step and the first of the next.  An empty
  // statement that reads the value keeps the shift (and the wait for the word) in the slot it is written in.
  auto pin_here = [](int v) { asm volatile("" : : "v"(v)); };
  static_assert((TM == 8 || TM == 4) && (TN == 8 || TN == 4), "wave tile is 128 or 64 rows/columns");

  // Software pipeline.  Ring slot s holds K-step ks with ks % NST == s.  The TM x TN grid of MFMAs
  // of a step is cut into four quadrants over the fragment halves lo = [0, H) and hi = [H, 2H),
  // issued in the order (a half, b half)
  //                      (lo,hi) (lo,lo) | (hi,hi) (hi,lo)
  // A step starts with a[lo] and b[hi] in registers.  During the first two quadrants it pulls
  // b[lo] and a[hi] out of its slot; after them every fragment of the step is in registers,
  // nobody needs the slot any more, and the step's one barrier sits THERE (the bar), in the
  // middle of the MFMA stream, with the wait for step ks+1 to have landed.  Behind it a[lo] is
  // dead, and after the third quadrant so is b[hi]: the wave reloads them with the fragments of
  // step ks+1 and slips the global->LDS loads of step ks+NST into the slot just released.  The
  // scale words of a half travel with its fragments: read at the start of a quadrant, shifted
  // into place at its end.  So LDS reads are spread evenly over the step (one fragment per four
  // MFMAs), every fragment is requested at least a quadrant before its first use, no register
  // is needed twice, and the MFMA pipe never drains at the barrier.  With one wave per SIMD
  // nothing else would hide those latencies.  sched_barrier pins the order (the compiler
  // otherwise sinks MFMAs below waits and barriers).
  static_assert(NST >= 2 && TM % 2 == 0 && TN % 2 == 0 && TM >= TN, "pipeline shape");
  constexpr std::true_type kBytes{};
  constexpr std::false_type kWords{};
  constexpr std::integral_constant<int, 0> kLo{};
  constexpr std::integral_constant<int, HA> kHiA{};
  constexpr std::integral_constant<int, HB> kHiB{};
  constexpr int S = HA * HB;  // MFMA time slots per quadrant
  // The scale values of a half are put in place one tile per time slot, in the slots that end with
  // kScaleLast (not the quadrant's last: what follows a step's last MFMA runs with the MFMA pipe idle),
  // from words or bytes requested in slot kScaleRead (words: slot 0).
  constexpr int kScaleLast = S >= 8 ? S - 2 : S - 1, kScaleRead = S >= 8 ? 1 : 0;
#pragma unroll
  for (int p = 0; p < NST; ++p) fetch(p < k_steps ? p : k_steps - 1, (uint32_t)(p * kStageBytes));
#pragma unroll
  for (int p = 0; p < kTouchAhead; ++p) touch(NST + p);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 1) * kLoadsPerStep + kTouchAhead * kTouch) : "memory");
  __syncthreads();
  if constexpr (KTAIL) {
    if (tail_step == 0) {  // a single, partly filled step: its scales are read next
      mask_tail_scales(0u);
      __syncthreads();
    }
  }
  const int a_row0 = wm * WM, b_row0 = wn * WN;
  // only the wave's first row differs between waves: fold it into the per-lane bases
  const uint32_t lane_lo_a = frag_lo + (a_row0 >> 3) * kGroupStride, lane_hi_a = frag_hi + (a_row0 >> 3) * kGroupStride;
  const uint32_t lane_lo_b = frag_lo + (b_row0 >> 3) * kGroupStride, lane_hi_b = frag_hi + (b_row0 >> 3) * kGroupStride;
  // with 4 tiles per wave the wave sits in the lower or upper 8 bytes of the 16-byte scale groups
  const uint32_t sc_lane_a = ((a_row0 & ~127) >> 7) * 512 + l16 * 16 + kOffSA + ((TM == 4 && (wm & 1)) ? 8 : 0);
  const uint32_t sc_lane_b = ((b_row0 & ~127) >> 7) * 512 + l16 * 16 + kOffSB + ((TN == 4 && (wn & 1)) ? 8 : 0);
  Frag fa[TM], fb[TN];
  int sa[KC][TM], sb[KC][TN];
  {
    const HalfWords wa = read_half_scales(kHiA, sc_lane_a, 0, kWords), wb = read_half_scales(kHiB, sc_lane_b, 1, kWords);
#pragma unroll
    for (int t = 0; t < HA; ++t) {
      fa[t] = load_frag(lane_lo_a, lane_hi_a, 0, t * 16);
#pragma unroll
      for (int c = 0; c < KC; ++c) sa[c][t] = scale_bits(wa.w[c][t], c, 0);
    }
#pragma unroll
    for (int t = 0; t < HB; ++t) {
      fb[HB + t] = load_frag(lane_lo_b, lane_hi_b, kOffB, (HB + t) * 16);
#pragma unroll
      for (int c = 0; c < KC; ++c) sb[c][HB + t] = scale_bits(wb.w[c][t], c, 0);
    }
  }

  // every refill of the loop is the partly filled step (the loop clamps a refill at the last step)
  if constexpr (KTAIL) {
    if (tail_step >= 0 && tail_step < NST) tail_in_place();
  }
  const uint64_t t_loop = clock_reading();
  // What a step needs of its ring slot `cur` and of the next step's `nxt`: the slots' offsets and the
  // per-lane fragment and scale addresses in them.  They are carried from step to step (this step's
  // `nxt` set is the next step's `cur` set) and the new `nxt` set is worked out in the middle of the
  // step's MFMA stream: whatever sits between the last MFMA of a step and the first of the next runs
  // with the MFMA pipe idle.
  uint32_t cur = 0, nxt = kStageBytes;  // NST >= 2
  uint32_t cla = lane_lo_a, cha = lane_hi_a, clb = lane_lo_b, chb = lane_hi_b, csa = sc_lane_a, csb = sc_lane_b;
  int ks = 0;
  do {  // k_steps >= 1
    if constexpr (KTAIL) {
      if (ks + NST == tail_step) tail_in_place();  // from this step's refill on
    }
    uint32_t nla, nha, nlb, nhb, nsa, nsb, nxt2;
    // the bases of step ks + NST, the refill of `cur` (clamped at the end: ignored), and the address of
    // the touch: scalar bookkeeping of the step's second half, done in slots of the first quadrant
    // that have nothing else to do, one item per slot
    StepBases at;
    const uint8_t* touch_p;
    constexpr int kBook = S >= 8 ? 2 : S - 2;  // first of those slots (a short quadrant takes it all in one)
    constexpr int kBookStep = S >= 8 ? 1 : 0;
    int n_dma = 0;
    bool touched = false;
    HalfWords hw;  // scale words of the half a quadrant brings in
    __builtin_amdgcn_sched_barrier(0);
    // MFMAs over a tiles i0.., b tiles j0.. with the b tile as the outer index (the b half of a
    // step's first quadrant is the one requested last); with FP4 first all tiles with the first
    // 128 elements of the step, then all with the second, so that the two MFMAs into one
    // accumulator are 16 apart.  `after(q)` follows the last MFMA of time slot q (one e4m3 MFMA
    // or two e2m1 MFMAs, the same number of cycles).
    auto quadrant = [&](auto i0_tag, auto j0_tag, auto&& after) {
      constexpr int i0 = decltype(i0_tag)::value, j0 = decltype(j0_tag)::value;
#pragma unroll
      for (int q = 0; q < S * KC; ++q) {
        const int c = q / S, t = q % S;
        const int i = i0 + t % HA, j = j0 + t / HA;
        // B fragment as the row operand: acc[i][j][v] = D[m = l16][n = 4*kq + v] of the tile
        if constexpr (!FP4) {
          const v8i vb = __builtin_shufflevector(fb[j].lo, fb[j].hi, 0, 1, 2, 3, 4, 5, 6, 7);
          const v8i va = __builtin_shufflevector(fa[i].lo, fa[i].hi, 0, 1, 2, 3, 4, 5, 6, 7);
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb, va, acc[i][j], 0, 0, 0, sb[0][j], 0, sa[0][i]);
        } else {
          // Written as assembly with the accumulator tied in place: left to the register
          // allocator, the two MFMAs per accumulator and step end up with different source
          // and destination registers and copies through VGPRs (60 moves per step).
          const v4i pb = c == 0 ? fb[j].lo : fb[j].hi, pa = c == 0 ? fa[i].lo : fa[i].hi;
          asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
                       : "+a"(acc[i][j])
                       : "v"(pb), "v"(pa), "v"(sb[c][j]), "v"(sa[c][i]));
        }
        if (q % KC == KC - 1) after(q / KC);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    auto dma = [&]() {
      if (n_dma < kLoadsPerStep) fetch_one(n_dma++, at, cur, 0u);
    };
    // e4m3: the step's loads (stage refill, then the touch as the youngest) are spread evenly over the 2 S
    // slots behind the bar: a wave gets one such load out per 40-odd cycles, so two of them in neighbouring
    // slots of 32 cycles hold the second one's slot up (issued in runs of two to five they cost 120 cycles a
    // step).  e2m1 keeps them out of the slots that request a fragment instead (measured both ways).
    auto vm_ops_of_slot = [&](int slot) {  // slot: 0 .. 2 S - 1
#pragma unroll
      for (int i = 0; i < kVmPerStep; ++i) {
        if ((i * 2 * S) / kVmPerStep != slot) continue;
        if (i < kLoadsPerStep) dma();
        else { touch_at(touch_p); touched = true; }
      }
    };
    // ---- before the bar: (lo,hi) pulls b[lo], (lo,lo) pulls a[hi], both from this step's slot
    // (a quadrant has S = HA * HB time slots; the HB fragments of a b half are requested every
    // HA slots, the HA fragments of an a half spread evenly over the quadrant)
    constexpr int kStepA = S / HA > 1 ? S / HA - 1 : 1;  // slots between two a fragments (4 x 4 tiles: 0, 3, 6, 9)
    quadrant(kLo, kHiB, [&](int q) {
      if (q == kScaleRead) hw = read_half_scales(kHiB, csb, 0, kBytes);  // slot 0 has a fragment request
      const int kn = ks + NST < k_steps ? ks + NST : k_steps - 1;
      if (q == kBook) { at.a = base_a(kn); asm volatile("" : : "s"(at.a)); }
      if (q == kBook + kBookStep) { at.b = base_b(kn); asm volatile("" : : "s"(at.b)); }
#pragma unroll
      for (int c = 0; c < KC; ++c)
        if (q == kBook + (2 + c) * kBookStep) { at.s[c] = base_s(kn, c); asm volatile("" : : "s"(at.s[c])); }
      if (TOUCH && q == kBook + (2 + KC) * kBookStep) { touch_p = touch_address(ks + NST + kTouchAhead); asm volatile("" : : "v"(touch_p)); }
      if (q % HA == 0) fb[q / HA] = load_frag(clb, chb, kOffB, (q / HA) * 16);
      if (const int t = q - (kScaleLast - HB + 1); t >= 0 && t < HB) {
#pragma unroll
        for (int c = 0; c < KC; ++c) sb[c][t] = FP4 ? scale_bits(hw.w[c][t], c, ks) : (int)hw.w[c][t];
      }
    });
    quadrant(kLo, kLo, [&](int q) {
      if (q == kScaleRead) hw = read_half_scales(kHiA, csa, 1, kBytes);
      if (q % kStepA == 0 && q / kStepA < HA) fa[HA + q / kStepA] = load_frag(cla, cha, 0, (HA + q / kStepA) * 16);
      if (const int t = q - (kScaleLast - HA + 1); t >= 0 && t < HA) {
#pragma unroll
        for (int c = 0; c < KC; ++c) sa[c][HA + t] = FP4 ? scale_bits(hw.w[c][t], c, ks) : (int)hw.w[c][t];
      }
      if (q == S - 3) {
        nla = nxt + lane_lo_a; nha = nxt + lane_hi_a; nlb = nxt + lane_lo_b; nhb = nxt + lane_hi_b;
      }
      if (q == S - 2) {
        nsa = nxt + sc_lane_a; nsb = nxt + sc_lane_b;
        nxt2 = nxt + kStageBytes == NST * kStageBytes ? 0u : nxt + kStageBytes;
      }
    });
    // every fragment of this step has been requested; once they are in, the slot is free
    // (the queue holds, in issue order, per step in flight its stage loads and then its touch
    // load: all but the loads of step ks+1 and whatever precedes them may stay outstanding.  The
    // touch has to stay the youngest: it misses the L2 by design, and loads complete in order)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_waitcnt vmcnt(%0)" ::"n"((NST - 2) * kVmPerStep + kTouch) : "memory");
    __syncthreads();
    if constexpr (KTAIL) {
      if (ks + 1 == tail_step) {  // the partly filled last step has landed: nobody has read its scales yet
        mask_tail_scales(nxt);
        __syncthreads();
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- behind the bar: (hi,hi) reloads a[lo], (hi,lo) reloads b[hi], both from step ks+1
    constexpr int kFirstFrag = HA > 2 ? 1 : 0;  // a[lo] fragments at kFirstFrag + k * kFragEvery, DMA loads in between
    constexpr int kFragEvery = HA > 2 ? (HB >= 4 ? 3 : 2) : 1;
    static_assert(kFirstFrag + (HA - 1) * kFragEvery < S, "the a[lo] reloads fit the quadrant");
    quadrant(kHiA, kHiB, [&](int q) {
      if (q == 0) hw = read_half_scales(kHiA, nsa, 0, kWords);
      const int f = (q - kFirstFrag) / kFragEvery;
      const bool frag_slot = q >= kFirstFrag && (q - kFirstFrag) % kFragEvery == 0 && f < HA;
      if (frag_slot) fa[f] = load_frag(nla, nha, 0, f * 16);
      if constexpr (!FP4) vm_ops_of_slot(q);
      else if (!frag_slot && q >= 1) dma();  // e2m1: two free issue slots per MFMA, so never next to a fragment request
      if (const int t = q - (kScaleLast - HA + 1); t >= 0 && t < HA) {
#pragma unroll
        for (int c = 0; c < KC; ++c) {
          sa[c][t] = scale_bits(hw.w[c][t], c, ks + 1);
          pin_here(sa[c][t]);
        }
      }
    });
    // (the last fragment is requested well before the step ends: what is still in flight at the loop's
    // back edge is waited for in full there)
    constexpr int kStepB = HB >= 4 ? 3 : HA;  // slots between two b fragments
    static_assert((HB - 1) * kStepB < S, "the b[hi] reloads fit the quadrant");
    quadrant(kHiA, kLo, [&](int q) {
      if (q == 0) hw = read_half_scales(kHiB, nsb, 1, kWords);
      const bool frag_slot = q % kStepB == 0 && q / kStepB < HB;
      if (frag_slot) fb[HB + q / kStepB] = load_frag(nlb, nhb, kOffB, (HB + q / kStepB) * 16);
      if constexpr (!FP4) vm_ops_of_slot(S + q);
      else if (frag_slot) {}
      else if (q == S - 3 && n_dma >= kLoadsPerStep) { touch_at(touch_p); touched = true; }
      else dma();
      if (const int t = q - (kScaleLast - HB + 1); t >= 0 && t < HB) {
#pragma unroll
        for (int c = 0; c < KC; ++c) {
          sb[c][HB + t] = scale_bits(hw.w[c][t], c, ks + 1);
          pin_here(sb[c][HB + t]);
        }
      }
    });
#pragma unroll
    for (int t = 0; t < kLoadsPerStep; ++t) dma();
    if (!touched) touch_at(touch_p);
    cur = nxt; nxt = nxt2;
    cla = nla; cha = nha; clb = nlb; chb = nhb; csa = nsa; csb = nsb;
  } while (++ks < k_steps);
  // the clamped refills of the last steps may still be landing: the epilogue reuses the LDS
  // (the no-ops cover the distance an assembly-written MFMA needs before its result is read)
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const uint64_t t_loop_end = clock_reading();

  if constexpr (SPLIT) {
    __shared__ uint32_t drawn;
    const int tile_id = tile_m * tiles_n + tile_n;
    const size_t per_split = (size_t)nb * (kWaves * TM * TN * kWave);  // accumulators (4 floats each) per split
    // a wave's 16 x 16 tile is two planes of 64 x 8 bytes (the accumulator's first and second pair
    // of floats), so that each 8-byte store instruction writes 512 contiguous bytes
    uint64_t* const mine = reinterpret_cast<uint64_t*>(partial + ((size_t)tile_id * kWaves + wave) * (TM * TN * kWave)) + lane;
    // 16 x 16 tiles wholly outside the matrix are neither parked nor added (uniform per wave)
    auto inside = [&](int i, int j) { return m0 + wm * WM + i * 16 < M && n0 + wn * WN + j * 16 < N; };
    typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
    auto park = [](uint64_t* q, v4f v) {
      const u64x2 w = __builtin_bit_cast(u64x2, v);
      __hip_atomic_store(q, w.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(q + kWave, w.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    auto fetch_parked = [](const uint64_t* q) -> v4f {
      u64x2 w;
      w.x = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      w.y = __hip_atomic_load(q + kWave, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return __builtin_bit_cast(v4f, w);
    };
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        if (inside(i, j)) park(mine + (split * per_split + (i * TN + j) * kWave) * 2, acc[i][j]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the parked values have arrived before the ticket is drawn
    __syncthreads();
    if (tid == 0) drawn = __hip_atomic_fetch_add(tickets + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (drawn != (uint32_t)(splits - 1)) return;
    if (tid == 0) tickets[tile_id] = 0u;  // every split has drawn: ready for the next launch
    // The loads of kBatch splits first, then the additions in split order: a round trip to memory
    // per kBatch splits, not one per split and tile.  The workgroup's own share is read back like
    // the others (the same bits as in its registers), which keeps the loop free of selects; tiles
    // outside the matrix and splits past the last add zeros.
    constexpr int kBatch = 4;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int sp0 = 0; sp0 < splits; sp0 += kBatch) {
      v4f p[kBatch][TM][TN];
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            p[u][i][j] = v4f{0.f, 0.f, 0.f, 0.f};
            if (sp0 + u < splits && inside(i, j))
              p[u][i][j] = fetch_parked(mine + ((sp0 + u) * per_split + (i * TN + j) * kWave) * 2);
          }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] += p[u][i][j];
    }
    __syncthreads();  // `drawn` and the epilogue staging share no bytes, but keep the waves together
  }

  // ---- epilogue: fp32 -> bf16 (v_cvt_pk_bf16_f32, round to nearest even) and out through LDS.
  // A lane holds 4 consecutive columns of one row per tile; written straight to memory that is
  // 32-byte pieces of 16 different rows per store.  Instead every wave parks its WM x WN tile
  // in its own LDS region (row pitch WN*2 + 16 bytes: conflict-free 8-byte writes) and reads
  // it back as 16 bytes per lane, 16 lanes per row, so a store instruction writes whole
  // 256-byte row segments.  The loop's last barrier has already retired every panel read.
  constexpr int kEpiPitch = WN * 2 + 16;
  uint8_t* epi = lds + wave * (WM * kEpiPitch);
  // rows 16 i0 .. 16 i1 of the wave's tile: convert and park
  auto park_rows = [&](int i0, int i1) {
#pragma unroll
    for (int i = i0; i < i1; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        u32x2 w;
        w.x = pack_bf16x2(acc[i][j].x, acc[i][j].y);
        w.y = pack_bf16x2(acc[i][j].z, acc[i][j].w);
        *reinterpret_cast<u32x2*>(epi + (i * 16 + l16) * kEpiPitch + (j * 16 + kq * 4) * 2) = w;
      }
  };
  constexpr int kChunksPerRow = WN * 2 / 16;             // 16-byte chunks per tile row
  constexpr int kRowsPerPass = kWave / kChunksPerRow;    // rows one store instruction covers
  const int erow = lane / kChunksPerRow, echunk = lane % kChunksPerRow;
  const int n = n0 + wn * WN + echunk * 8;
  // a tile wholly inside the matrix with an aligned output (the common case): no edge tests, the
  // row pointer moves by a constant
  if (wide_stores && m0 + BM <= M && n0 + BN <= N) {
    // one 16-row strip of the wave's tile at a time, so that a strip's stores are on their way while the
    // next one is converted (a wave only touches its own region: no barrier, the LDS counter orders the
    // reads behind the writes).  8192^3, us per launch on constant / random operands: all rows parked
    // first 278.3 / 380.6, in halves 276.0 / -, in quarters 274.8 / 377.8, by strips 274.3 / 376.2
    // (without any epilogue the launch takes 259 / 352: 12 of those 19 us are the stores)
    uint16_t* dst = out + (int64_t)(m0 + wm * WM + erow) * ldo + n;
    const int64_t pass_stride = (int64_t)kRowsPerPass * ldo;
    const uint8_t* src = epi + erow * kEpiPitch + echunk * 16;
    constexpr int kEpiParts = TM;
    constexpr int kHalfTiles = TM / kEpiParts, kHalfRows = WM / kEpiParts;
    static_assert(kHalfRows % kRowsPerPass == 0, "a store pass stays inside a part");
#pragma unroll
    for (int half = 0; half < kEpiParts; ++half) {
      park_rows(half * kHalfTiles, (half + 1) * kHalfTiles);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = half * kHalfRows; r < (half + 1) * kHalfRows; r += kRowsPerPass) {
        *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(src + r * kEpiPitch);
        dst += pass_stride;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (kPhaseLog && phase_log) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (threadIdx.x == 0) {
        uint64_t* const e = phase_log + (size_t)blockIdx.x * 8;
        e[0] = t_start; e[1] = t_loop; e[2] = t_loop_end; e[3] = wall_clock64();
        e[4] = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (31 << 11));  // XCC_ID
        e[5] = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | (31 << 11));   // HW_ID
      }
    }
    return;
  }
  park_rows(0, TM);
#pragma unroll
  for (int r = 0; r < WM; r += kRowsPerPass) {
    const int row = r + erow;
    const int m = m0 + wm * WM + row;
    if (m >= M || n >= N) continue;
    const u32x4 v = *reinterpret_cast<const u32x4*>(epi + row * kEpiPitch + echunk * 16);
    uint16_t* dst = out + (int64_t)m * ldo + n;
    if (wide_stores && n + 8 <= N) {
      *reinterpret_cast<u32x4*>(dst) = v;
    } else {  // N % 4 == 0 is checked on the host: a chunk is 8 or 4 valid columns
      *reinterpret_cast<u32x2*>(dst) = u32x2{v.x, v.y};
      if (n + 8 <= N) *reinterpret_cast<u32x2*>(dst + 4) = u32x2{v.z, v.w};
    }
  }
}

// blocks > 0: launch only that many workgroups (the first `blocks` of the tiling, or with kQuads the
// quadrants of `blocks` 256 x 256 tiles from tile number first_block on)
template <int BM, int BN, int WAVES_M, int WAVES_N, int NST, bool FP4, bool TOUCH, int MODE, bool KTAIL>
int launch_gemm_impl(const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M, int64_t N,
                int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo, hipStream_t stream, int splits,
                void* workspace, int64_t blocks, int first_block) {
  constexpr bool kParts = MODE == kQuads || MODE == kHalves;
  constexpr int kTileM = kParts ? 256 : BM, kTileN = kParts ? 256 : BN;
  const int tiles_m = (int)ceil_div(M, kTileM), tiles_n = (int)ceil_div(N, kTileN);
  if ((int64_t)tiles_m * tiles_n > 0x7FFFFFFFll) return DT_ERR_INVALID_SHAPE;  // one workgroup per tile
  // NST K-steps: panels + scale slots (1 KiB per operand and 128-element chunk of the step)
  size_t lds_bytes = (size_t)NST * (((BM + BN) / kGroupRows) * kGroupStride + 2048 * (FP4 ? 2 : 1));
  const size_t epi_bytes = (size_t)WAVES_M * WAVES_N * (BM / WAVES_M) * ((BN / WAVES_N) * 2 + 16);  // epilogue staging
  if (TOUCH) lds_bytes += 256;  // dump area of the L2 prefetch loads
  if (lds_bytes < epi_bytes) lds_bytes = epi_bytes;
  // A grid that fits the chip once should land one workgroup per CU: asking for more than half
  // of the LDS keeps the dispatcher from pairing two workgroups on one CU while others idle.
  if ((int64_t)tiles_m * tiles_n * splits <= device_facts().cu_count && lds_bytes < 82 * 1024) lds_bytes = 82 * 1024;
  auto kernel = mx_gemm_kernel<BM, BN, WAVES_M, WAVES_N, NST, FP4, TOUCH, MODE, KTAIL>;
  if (lds_bytes > 64 * 1024) {
    // once per instantiation and device, with the largest size asked for so far (a host call per launch otherwise)
    static std::atomic<int> allowed[16];
    int dev = 0;
    (void)hipGetDevice(&dev);
    const bool tracked = dev >= 0 && dev < 16;
    if (!tracked || allowed[dev].load(std::memory_order_relaxed) < (int)lds_bytes) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds_bytes) != hipSuccess)
        return DT_ERR_LAUNCH;
      if (tracked) allowed[dev].store((int)lds_bytes, std::memory_order_relaxed);
    }
  }
  uint8_t* const ws = static_cast<uint8_t*>(workspace);  // ticket counters, then the parked accumulators
  int64_t grid = (int64_t)tiles_m * tiles_n * splits;
  if (blocks > 0) grid = kParts ? (MODE == kQuads ? 32 : 16) * ceil_div(blocks, (int64_t)8) : blocks;
  kernel<<<(unsigned)grid, WAVES_M * WAVES_N * kWave, lds_bytes, stream>>>(
      a, b, sfa, sfb, (int)M, (int)N, (int)K, lda, ldb, static_cast<uint16_t*>(out), ldo, tiles_m, tiles_n,
      (ldo % 8 == 0 && aligned(out, 16)) ? 1 : 0, splits, ws ? reinterpret_cast<v4f*>(ws + kSplitTicketBytes) : nullptr,
      reinterpret_cast<uint32_t*>(ws), first_block, phase_log((size_t)grid * 64));
  return launch_status();
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int NST, bool FP4, bool TOUCH, int MODE = kPlain>
int launch_gemm(const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M, int64_t N,
                int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo, hipStream_t stream, int splits = 1,
                void* workspace = nullptr, int64_t blocks = 0, int first_block = 0) {
  const int64_t k_bytes = FP4 ? K / 2 : K;
  if (k_bytes % kBK != 0)  // a partly filled last step: the build of the kernel that deals with it
    return launch_gemm_impl<BM, BN, WAVES_M, WAVES_N, NST, FP4, TOUCH, MODE, true>(a, b, sfa, sfb, M, N, K, lda, ldb, out, ldo, stream,
                                                                                 splits, workspace, blocks, first_block);
  return launch_gemm_impl<BM, BN, WAVES_M, WAVES_N, NST, FP4, TOUCH, MODE, false>(a, b, sfa, sfb, M, N, K, lda, ldb, out, ldo, stream,
                                                                                splits, workspace, blocks, first_block);
}

inline size_t split_workspace_bytes() { return kSplitTicketBytes + (size_t)device_facts().cu_count * kSplitTileBytes; }

// Split-K factor for the 128 x 128 tiling.  A grid of a third of a workgroup per CU or less leaves
// most of the chip idle while each workgroup walks the whole K, one K-step per memory latency / 3:
// share K between as many workgroups per tile as fill the chip once.  What it costs is the last
// workgroup of a tile reading every share through one CU (about 1 us per share of a full tile),
// so a share is at least 16 K-steps and two shares are not worth it (measured on MI355X, e4m3,
// us without -> with: 16 x 8192 x 8192 31 -> 19, 128 x 8192 x 8192 31 -> 24, 1024 x 1024 x 16384
// 58 -> 34, 512 x 512 x 65536 219 -> 50, 128 x 128 x 16384 56 -> 25; no gain: 256 x 8192 x 8192 with
// two shares 31.5 -> 32.4, 1024 x 1024 x 4096 with four shares of 8 steps 18.3 -> 19.3).  The knob
// gemm.split_k forces a factor (1 = never split); whatever is asked for, every split owns a step
// and the workspace holds all shares.
inline int plan_splits(int64_t M, int64_t N, int64_t k_steps, size_t workspace_bytes) {
  const int64_t tiles = ceil_div(M, 128) * ceil_div(N, 128);
  if (workspace_bytes <= kSplitTicketBytes || tiles > (int64_t)(kSplitTicketBytes / 4)) return 1;
  const int64_t room = (int64_t)((workspace_bytes - kSplitTicketBytes) / kSplitTileBytes) / tiles;
  const int forced = tuning("gemm.split_k");
  int64_t want;
  if (forced > 0) {
    want = forced;
  } else {
    const int cus = device_facts().cu_count;
    if (tiles * 3 > cus) return 1;
    want = cus / tiles;
    if (want > k_steps / 16) want = k_steps / 16;
    if (want > kAutoMaxSplits) want = kAutoMaxSplits;
    if (want < 3) return 1;
  }
  if (want > kMaxSplits) want = kMaxSplits;
  if (want > room) want = room;
  if (want > k_steps) want = k_steps;
  if (want < 2) return 1;
  const int64_t per = ceil_div(k_steps, want);
  return (int)ceil_div(k_steps, per);
}

// Shared argument checks and tile choice.  K counts elements, lda/ldb bytes.
template <bool FP4>
int mx_gemm(const void* a, const void* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M, int64_t N, int64_t K,
            int64_t lda, int64_t ldb, void* out, int64_t ldo, void* workspace, size_t workspace_bytes,
            dt_stream_t stream) {
  if (M < 0 || N < 0 || K < 0) return DT_ERR_INVALID_SHAPE;
  if (M == 0 || N == 0) return DT_OK;
  if (K == 0 || K % 32 != 0) return DT_ERR_INVALID_SHAPE;  // whole MX blocks
  const int64_t k_bytes = FP4 ? K / 2 : K;
  if (N % 4 != 0 || ldo % 4 != 0 || ldo < N || lda < k_bytes || ldb < k_bytes) return DT_ERR_INVALID_SHAPE;
  if (M > 0x7FFFFF00ll || N > 0x7FFFFF00ll || K > 0x7FFFFF00ll) return DT_ERR_INVALID_SHAPE;
  if (!a || !b || !sfa || !sfb || !out) return DT_ERR_NULL_POINTER;
  if (!aligned(a, 16) || !aligned(b, 16) || lda % 16 != 0 || ldb % 16 != 0) return DT_ERR_MISALIGNED;
  if (!aligned(out, 8) || !aligned(sfa, 4) || !aligned(sfb, 4)) return DT_ERR_MISALIGNED;
  if (workspace && !aligned(workspace, 256)) return DT_ERR_MISALIGNED;
  // per-lane byte offsets are 32 bits wide and span the rows of one tile (at most 256)
  if (255 * lda + k_bytes + 3 * 1024 > 0xFFFFFFFFll || 255 * ldb + k_bytes + 3 * 1024 > 0xFFFFFFFFll) return DT_ERR_INVALID_SHAPE;  // + the bias of a run of loads
  const uint8_t* A = static_cast<const uint8_t*>(a);
  const uint8_t* B = static_cast<const uint8_t*>(b);
  hipStream_t s = as_hip(stream);
  const int variant = tuning("gemm.variant");
  if ((variant == 9 && few_rows_fits(M, K)) || (variant == 0 && few_rows_pays(FP4, M, N, K, workspace != nullptr)))
    return launch_few_rows(FP4, A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s);
  const int64_t tiles256 = ceil_div(M, 256) * ceil_div(N, 256);
  const bool big = variant == 2 || variant == 7 || (variant == 0 && tiles256 >= device_facts().cu_count / 2);
  // <tile M, tile N, waves M, waves N, LDS ring slots, e2m1 operands>
  if (big && variant == 7) return launch_gemm<256, 256, 2, 2, 2, FP4, false>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s);
  // Between a quarter and half a round of 256 x 256 tiles: as 256 x 128 halves they fill the chip
  // once (0.8 of a round of tiles), as 128 x 128 tiles they would take two rounds (2 x 0.55)
  if (variant == 0 && tuning("gemm.tail_quads") != 0 && 4 * tiles256 > device_facts().cu_count &&
      2 * tiles256 <= device_facts().cu_count)
    return launch_gemm<256, 128, 2, 2, 3, FP4, false, kHalves>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s, 1, nullptr,
                                                               tiles256, 0);
  if (big) {
    // Whole rounds of the chip on 256 x 256 tiles; what is left over would keep the chip for another
    // full round however few tiles it is.  When its quadrants fit the chip at once it runs as
    // 128 x 128 quadrants instead: one round of those takes 0.5-0.6 of a round of tiles (measured on
    // MI355X, e4m3, us: 4096 x 5120 x 4096, 256 + 64 tiles, 97 -> 77; 4352^2 x 4096, 256 + 33, 97 -> 78;
    // 4096 x 4352 x 8192, 256 + 16, 177 -> 134; 6144^3, 512 + 64, 216 -> 186; 8448 x 8192^2, 1024 + 32,
    // 473 -> 436), two rounds of quadrants take as long as the round of tiles (4096 x 6144 x 4096,
    // 256 + 128: 97 -> 96).  Up to half a round of leftover tiles runs as 256 x 128 halves, a round of
    // which takes 0.8 of a round of tiles (the same shape 97 -> 87.5; 8192 x 5120 x 8192, 512 + 128,
    // 273 -> 258).  The results are the same bits either way.
    const int cus = device_facts().cu_count;
    const int64_t rounds = tiles256 / cus, left = tiles256 % cus;
    const int tail = tuning("gemm.tail_quads");
    if (variant == 0 && tail != 0 && rounds >= 1 && left > 0 && cus % 8 == 0 && (tail >= 2 || 2 * left <= cus)) {
      const int st = launch_gemm<256, 256, 2, 2, 2, FP4, true>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s, 1, nullptr,
                                                                rounds * cus);
      if (st != DT_OK) return st;
      if (tail == 2 || (tail == 1 && 4 * left <= cus))
        return launch_gemm<128, 128, 2, 2, 4, FP4, false, kQuads>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s, 1, nullptr,
                                                                  left, (int)(rounds * cus));
      return launch_gemm<256, 128, 2, 2, 3, FP4, false, kHalves>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s, 1, nullptr,
                                                                 left, (int)(rounds * cus));
    }
    return launch_gemm<256, 256, 2, 2, 2, FP4, true>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s);
  }
  const int splits = workspace ? plan_splits(M, N, ceil_div(k_bytes, (int64_t)kBK), workspace_bytes) : 1;
  if (splits > 1)
    return launch_gemm<128, 128, 2, 2, 4, FP4, false, kSplitK>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s, splits, workspace);
  return launch_gemm<128, 128, 2, 2, 4, FP4, false>(A, B, sfa, sfb, M, N, K, lda, ldb, out, ldo, s);
}

}  // namespace dt
