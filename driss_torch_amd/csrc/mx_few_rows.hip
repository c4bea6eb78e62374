// The block-scaled GEMM for few rows (M <= 64): out[M,N] = (A 2^sfa)(B 2^sfb)^T with e4m3 or e2m1 operands.
//
// Such a problem is one pass over B, and a tile with a 128- or 256-row A panel would idle most of its
// MFMAs and leave the chip to a handful of workgroups.  Here a workgroup of WAVES waves owns a group of
// 16 NT rows of B (= output columns) at a time and every row of A; its waves share K between them in
// turns of U K-steps of 128 elements, so the workgroup as a whole walks 16 NT whole rows of B.  Nothing
// goes through LDS on the way in: a lane's part of an MFMA operand is two 16-byte pieces of one row, 64
// bytes apart (one piece with e2m1), and the four lanes that share a row read 64 contiguous bytes of it
// per load instruction (bytes 16 g .. of the step in lane group g); the E8M0 byte of a lane is one byte of
// the blocked scale buffer.  A's rows come out of the L2 the same way (every workgroup reads all of A: M x K
// bytes, a few hundred KiB).  A batch of U steps is in registers while the next one's loads are in flight.
// The waves' partial sums meet in LDS and are added in wave order; one wave per 16 x 16 output tile writes
// it.  K-blocks past the end of K (K % 128 != 0) enter as zeros with a scale of 2^-127.
//
// The grid is persistent: a workgroup takes the column groups b, b + grid, ... and the batch it loads
// ahead may belong to its next group, so those loads are in flight under the reduction and the stores of
// the group in hand.
#include "mx_few_rows.hpp"

#include "dt_device.hpp"
#include "dt_host.hpp"

namespace dt {

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

template <bool FP4, int MT, int NT, int WAVES, int U>
__global__ __launch_bounds__(WAVES* kWave) void mx_few_rows_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                                                                  const uint8_t* __restrict__ sfa, const uint8_t* __restrict__ sfb,
                                                                  int M, int N, int K, int64_t lda, int64_t ldb,
                                                                  uint16_t* __restrict__ out, int64_t ldo, int groups, int stagger) {
  constexpr int kStepBytes = FP4 ? 64 : 128;  // bytes of a row that one MFMA takes
  static_assert(MT >= 1 && MT <= 4 && NT >= 1 && NT <= 2, "at most 64 rows of A, 32 columns per group");
  __shared__ v4f part[WAVES][MT * NT][kWave];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int l16 = lane & 15, g = lane >> 4;
  const int k_steps = (K + 127) / 128;  // = chunks of four scale bytes per row of the blocked buffers
  // Addresses are a base that is the same for the whole workgroup plus a 32-bit offset per lane (the
  // host has checked that 255 rows of an operand span less than 4 GiB).  A group's rows of B lie in one
  // 128-row chunk of the blocked scales, and all of A's rows in the first.
  auto scale_offset = [&](int row) { return (uint32_t)((row & 31) * 16 + ((row & 127) >> 5) * 4 + g); };
  uint32_t oa[MT], osa[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int arow = t * 16 + l16 < M ? t * 16 + l16 : M - 1;
    oa[t] = (uint32_t)arow * (uint32_t)lda + g * 16;
    osa[t] = scale_offset(arow);
  }
  // what of B depends on the column group
  struct Group {
    const uint8_t *b0, *sb0;
    uint32_t ob[NT], osb[NT];
  };
  auto group_at = [&](int grp) {
    Group q;
    const int n0 = grp * (16 * NT);
    q.b0 = b + (int64_t)n0 * ldb;
    q.sb0 = sfb + (int64_t)(n0 >> 7) * k_steps * 512;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int brow = n0 + j * 16 + l16 < N ? n0 + j * 16 + l16 : N - 1;  // rows past the edge re-read the last one; never stored
      q.ob[j] = (uint32_t)(brow - n0) * (uint32_t)ldb + g * 16;
      q.osb[j] = scale_offset(brow);
    }
    return q;
  };
  struct Batch {
    v4i blo[NT][U], bhi[NT][U], alo[MT][U], ahi[MT][U];
    int sb[NT][U], sa[MT][U];
  };
  const v4i zero4 = {0, 0, 0, 0};
#ifdef DT_FEW_ROWS_STREAM_B
  auto ld_b = [](const v4i* p) { return __builtin_nontemporal_load(p); };
#else
  auto ld_b = [](const v4i* p) { return *p; };
#endif
  auto load = [&](Batch& w, const Group& q, int first_step) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = first_step + u;
      // What of the step lies inside K.  The scale byte of lane group g is that of the step's K-block g;
      // its e2m1 elements are that block, but its e4m3 elements are the two 16-byte pieces at 16 g and
      // 64 + 16 g, which belong to K-blocks g / 2 and 2 + g / 2.
      const int left = K - k * 128;  // elements from this step on (none: the batch reaches past the last step)
      const bool valid = g * 32 < left;
      const bool valid_lo = FP4 ? valid : (g >> 1) * 32 < left, valid_hi = 64 + (g >> 1) * 32 < left;
      const uint8_t* const bk = q.b0 + (int64_t)k * kStepBytes;
      const uint8_t* const ak = a + (int64_t)k * kStepBytes;
      const uint8_t* const sbk = q.sb0 + (int64_t)k * 512;
      const uint8_t* const sak = sfa + (int64_t)k * 512;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        w.blo[j][u] = valid_lo ? ld_b(reinterpret_cast<const v4i*>(bk + q.ob[j])) : zero4;
        if constexpr (!FP4) w.bhi[j][u] = valid_hi ? ld_b(reinterpret_cast<const v4i*>(bk + 64 + q.ob[j])) : zero4;
        w.sb[j][u] = valid ? (int)sbk[q.osb[j]] : 0;
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        w.alo[t][u] = valid_lo ? *reinterpret_cast<const v4i*>(ak + oa[t]) : zero4;
        if constexpr (!FP4) w.ahi[t][u] = valid_hi ? *reinterpret_cast<const v4i*>(ak + 64 + oa[t]) : zero4;
        w.sa[t][u] = valid ? (int)sak[osa[t]] : 0;
      }
    }
  };
  v4f acc[MT][NT];
  auto clear = [&]() {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};
  };
  auto compute = [&](const Batch& w) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const v8i vb = FP4 ? __builtin_shufflevector(w.blo[j][u], zero4, 0, 1, 2, 3, 4, 5, 6, 7)
                           : __builtin_shufflevector(w.blo[j][u], w.bhi[j][u], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const v8i va = FP4 ? __builtin_shufflevector(w.alo[t][u], zero4, 0, 1, 2, 3, 4, 5, 6, 7)
                             : __builtin_shufflevector(w.alo[t][u], w.ahi[t][u], 0, 1, 2, 3, 4, 5, 6, 7);
          // B as the row operand: acc[t][j][v] = D[row 16 t + l16][column n0 + 16 j + 4 g + v]
          acc[t][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb, va, acc[t][j], FP4 ? 4 : 0, FP4 ? 4 : 0, 0,
                                                                       w.sb[j][u], 0, w.sa[t][u]);
        }
      }
  };
  // The end of a group: the waves' sums meet in LDS and are added in wave order (the same sum whatever
  // the timing); wave t takes the output tiles t, t + WAVES, ...
  auto finish = [&](int grp) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int j = 0; j < NT; ++j) part[wave][t * NT + j][lane] = acc[t][j];
    __syncthreads();
    const int n0 = grp * (16 * NT);
#pragma unroll
    for (int tile0 = 0; tile0 < MT * NT; tile0 += WAVES) {
      const int tile = tile0 + wave;
      if (tile < MT * NT) {
        v4f sum = part[0][tile][lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += part[w][tile][lane];
        const int m = (tile / NT) * 16 + l16, n = n0 + (tile % NT) * 16 + 4 * g;
        if (m < M && n < N)  // N % 4 == 0: four columns or none
          *reinterpret_cast<u32x2*>(out + (int64_t)m * ldo + n) = u32x2{pack_bf16x2(sum.x, sum.y), pack_bf16x2(sum.z, sum.w)};
      }
    }
    __syncthreads();  // before anybody parks the next group's sums
  };

  // This wave's batches of a group: wave, wave + WAVES, ... of U steps each.  The workgroups do not all
  // start at the front of their rows: group number grp begins `rot` batches in and wraps around, so that
  // at any moment the chip's loads are spread over the whole length of the rows (the rows are a power of
  // two apart in most problems: with every workgroup at the same K offset the requests of the moment
  // fall on a fraction of the memory channels).
  const int batches = (k_steps + U - 1) / U;
  auto first_step_of = [&](int grp, int i) {
    const int r = i + (stagger ? (int)(((unsigned)grp * 5u) % (unsigned)batches) : 0);
    return (r >= batches ? r - batches : r) * U;
  };
  // The sequence of (group, batch) pairs of this wave, over two register sets: the pair after the one
  // being computed is already on its way, also across the end of a group.
  int grp = blockIdx.x, bi = wave;
  auto advance = [&](int& gq, int& bq) {  // the pair after (gq, bq); gq >= groups: none
    bq += WAVES;
    if (bq >= batches) { bq = wave; gq += gridDim.x; }
  };
  if (wave >= batches) {  // fewer batches than waves: this wave only takes part in the reductions
    for (; grp < groups; grp += gridDim.x) { clear(); finish(grp); }
    return;
  }
  if (grp >= groups) return;  // (the whole workgroup)
  Batch wa, wb;
  Group q = group_at(grp);
  load(wa, q, first_step_of(grp, bi));
  clear();
  for (;;) {
    // ---- wa holds (grp, bi): send for its successor into wb, compute wa
    int g2 = grp, b2 = bi;
    advance(g2, b2);
    Group q2 = q;
    if (g2 != grp && g2 < groups) q2 = group_at(g2);
    if (g2 < groups) load(wb, q2, first_step_of(g2, b2));
    compute(wa);
    if (g2 != grp) { finish(grp); clear(); }
    if (g2 >= groups) break;
    grp = g2; bi = b2; q = q2;
    // ---- wb holds (grp, bi): the same with the roles of the sets swapped
    advance(g2, b2);
    if (g2 != grp && g2 < groups) q2 = group_at(g2);
    if (g2 < groups) load(wa, q2, first_step_of(g2, b2));
    compute(wb);
    if (g2 != grp) { finish(grp); clear(); }
    if (g2 >= groups) break;
    grp = g2; bi = b2; q = q2;
  }
}

// Shape of the launch for a problem: 16-column tiles per group (NT), waves per workgroup, K-steps per batch
struct Plan {
  int nt, waves, steps;
};

Plan plan_for(bool fp4, int64_t M, int64_t N) {
  Plan p;
  const int tiles = tuning("gemm.few_rows_tiles");
  p.nt = tiles ? (tiles == 2 ? 2 : 1) : (N >= 32 * (int64_t)device_facts().cu_count && (fp4 || M > 8) ? 2 : 1);
  const int mt = (int)((M + 15) / 16);
  const int waves = tuning("gemm.few_rows_waves");
  p.waves = waves == 4 ? 4 : 8;
  int steps = tuning("gemm.few_rows_steps");
  if (steps != 1 && steps != 2 && steps != 4) steps = mt == 1 ? (fp4 ? 4 : 2) : (p.nt == 2 && mt == 2) ? 2 : 1;
  // two register sets of (NT + MT) U fragments of 4 (e2m1) or 8 registers must leave room for the rest
  while (steps > 1 && 2 * (p.nt + mt) * steps * (fp4 ? 4 : 8) > 144) steps /= 2;
  p.steps = steps;
  return p;
}

}  // namespace

// Where the kernel above beats the tiles (measured on MI355X, us, few rows against 128 x 128 tiles with
// K shared through a workspace / without one; B rotated through 5 buffers so that it comes from HBM):
// e2m1 16 x 8192 x 8192 11.7 against 21.7, 32 rows 14.7, 64 rows 18.9 against 22.1, 16 x 2048 x 8192 10.7
// against 21.5, 16 x 16384 x 4096 11.4 against 13.0; e4m3 1 x 8192 x 8192 15.5 against 22.1 / 31.9,
// 16 rows 21.4 against 20.0 / 31.8, 32 rows 24.2 against 23.1 / 32.3, 64 rows 31.9 against 23.8 / 35.0.
// It loses where a workgroup reads more than twice as much of A as of B (64 x 4096 x 14336 e2m1: 25.6
// against 19.0), and for e4m3 against tiles that share K through a workspace.
bool few_rows_pays(bool fp4, int64_t M, int64_t N, int64_t K, bool have_workspace) {
  const int64_t cus = device_facts().cu_count;
  if (M > 64 || N < 8 * cus || K < 4096) return false;
  const Plan p = plan_for(fp4, M, N);
  if (M > 32 * p.nt) return false;
  return fp4 || !have_workspace || M <= 8;
}

int launch_few_rows(bool fp4, const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb, int64_t M, int64_t N,
                    int64_t K, int64_t lda, int64_t ldb, void* out, int64_t ldo, hipStream_t stream) {
  uint16_t* o = static_cast<uint16_t*>(out);
  const Plan p = plan_for(fp4, M, N);
  const int mt = (int)((M + 15) / 16);
  const int64_t groups = ceil_div(N, (int64_t)16 * p.nt);
  int per_cu = tuning("gemm.few_rows_per_cu");
  if (per_cu < 1) per_cu = 2;
  int64_t grid = groups;
  if (grid > (int64_t)device_facts().cu_count * per_cu) grid = (int64_t)device_facts().cu_count * per_cu;
  const int stagger = tuning("gemm.few_rows_stagger");
#define DT_FEW(FP4, MT, NT, WAVES, U)                                                                                    \
  mx_few_rows_kernel<FP4, MT, NT, WAVES, U><<<(unsigned)grid, WAVES * kWave, 0, stream>>>(a, b, sfa, sfb, (int)M, (int)N, (int)K, \
                                                                                       lda, ldb, o, ldo, (int)groups, stagger)
#define DT_FEW_U(FP4, MT, NT, WAVES)                                                      \
  do {                                                                                    \
    constexpr int kMaxU = 144 / (2 * (NT + MT) * (FP4 ? 4 : 8));                          \
    if constexpr (kMaxU >= 4) { if (p.steps == 4) { DT_FEW(FP4, MT, NT, WAVES, 4); break; } } \
    if constexpr (kMaxU >= 2) { if (p.steps >= 2) { DT_FEW(FP4, MT, NT, WAVES, 2); break; } } \
    DT_FEW(FP4, MT, NT, WAVES, 1);                                                        \
  } while (0)
#define DT_FEW_W(FP4, MT, NT) do { if (p.waves == 4) DT_FEW_U(FP4, MT, NT, 4); else DT_FEW_U(FP4, MT, NT, 8); } while (0)
#define DT_FEW_N(FP4, MT) do { if (p.nt == 2) DT_FEW_W(FP4, MT, 2); else DT_FEW_W(FP4, MT, 1); } while (0)
#define DT_FEW_M(FP4)                         \
  do {                                        \
    if (mt == 1) DT_FEW_N(FP4, 1);            \
    else if (mt == 2) DT_FEW_N(FP4, 2);       \
    else if (mt == 3) DT_FEW_N(FP4, 3);       \
    else DT_FEW_N(FP4, 4);                    \
  } while (0)
  if (fp4) DT_FEW_M(true);
  else DT_FEW_M(false);
#undef DT_FEW_M
#undef DT_FEW_N
#undef DT_FEW_W
#undef DT_FEW_U
#undef DT_FEW
  return launch_status();
}

}  // namespace dt
