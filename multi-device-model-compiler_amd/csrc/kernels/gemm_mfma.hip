// fp16 / bf16 GEMM with the bias, activation and residual epilogue fused, on
// gfx950 MFMA: out[M,N] = act(in[M,K] . W[K,N] + bias[N]) (+ residual[M,N]).
//
// One of the two ways mgpuMatmulEx<half> (lib/Kernels/GPU/Ops.cu:134-234) is
// served; the other is the library GEMM in gemm.cpp, and gemm.cpp times both
// on the first use of a shape.  This kernel exists for the shapes of a
// transformer layer at a few thousand tokens (M = 4096, N and K between 768
// and 3072), where a GEMM is a few hundred 128x128 tiles - one to three per
// CU - and the time goes to ramp-up, tail and the epilogue rather than to a
// long steady state; and for the exact-erf GELU, which the library cannot fuse.
//
// Work decomposition.  A 256-thread block (4 wavefronts) owns a 128 x 128 output
// tile (wavefronts 2 x 2, each 64 x 64 as 2 x 2 accumulators of 32 x 32) or a
// 128 x 96 one (wavefronts 4 x 1, each 32 x 96 as 3 accumulators); the launcher
// takes the width that loads the busiest CU least (768 columns are 6 tiles of
// 128 - 192 tiles at M = 4096, a quarter of the CUs idle - or 8 of 96 - 256
// tiles, one per CU).  The reduction runs in steps of 32: per step an 8 KiB
// slice of the input (128 rows of 64 bytes) and a slice of the weight (32 rows
// at a 256-byte pitch) travel HBM -> LDS directly (global_load_lds, 16 bytes per
// lane) into a ring of three stages, two steps in flight behind the one
// consumed; three blocks share a CU (48 KiB of LDS, < 128 VGPRs).  When there
// is at most one tile per CU the step is 64 instead (96 KiB of LDS) and the
// block has eight wavefronts: a lone block cannot hide the barrier and the LDS
// latency of a step behind other blocks, so it takes half as many, longer
// steps, and wavefronts 4-7 cover the tile like 0-3 but take the upper half of
// every step (all eight share the loads); the two sets of accumulators meet in
// LDS before the epilogue (4096 x 768 x 3072: 35.2 -> 30.2 us).  With several tiles per CU
// and K a multiple of 64 the input rows are fetched for two steps at a time
// (two buffers of 128 rows x 128 bytes, the weight slices in a ring of two):
// a 64-byte piece of a row is half a cache line, and fetched on its own it
// costs the whole line on the way from L2 (loads alone: 18.3 us against 21.7
// at 4096 x 3072 x 768).
//
// MFMA formulation: the transposed product out^T[n, m] = W^T[n, k] . in^T[k, m],
//   A operand = W^T: the weight slice sits in LDS row-major as in memory
//     ([k][n], n contiguous); ds_read_b64_tr_b16 hands lane (n = l % 32) the
//     four k of its column, two reads per operand;
//   B operand = in^T: lane (m = l % 32) reads 16 contiguous bytes of its row.
// so that an accumulator register group holds four consecutive n of one row m:
// bias, activation and residual are applied on 8-byte pieces of output rows,
// and the tile is then transposed through LDS so that every store instruction
// writes whole 128-byte runs of output rows.  Both slices are stored unpadded
// (the direct loads fill 1 KiB of consecutive LDS per instruction) with an XOR
// swizzle on the 16-byte chunk index that keeps both operand reads free of
// bank conflicts.
//
// Shapes: M a multiple of 128, N of 128 or 96, K of 32, 16-byte aligned
// operands.  Everything else goes to the library.
#include "common.hpp"
#include "mfma.hpp"
#include "mgpu_ops_internal.hpp"
#include "types.hpp"

namespace mgpu {

namespace {

typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kBM = 128;       // rows of an output tile
constexpr int kRing = 3;       // LDS ring depth
constexpr int kWRow = 256;     // LDS pitch of a weight-slice row, bytes (128 columns, of which NB * 32 are loaded)

// Chunk swizzles: the 16-byte chunk c of a row is kept at chunk c ^ swz(row).
template <int BK> __host__ __device__ constexpr int aSwz(int row) {
  return BK == 32 ? (row >> 2) & 3 : (row >> 1) & 7; // 4 or 8 chunks per row
}
__host__ __device__ constexpr int wSwz(int row) { return (row & 3) << 2; } // 16 chunks per row

// T: element type; ACT: epilogue activation; BK: reduction step (32 or 64);
// NB: tile width in 32-column blocks (4 or 3).
template <typename T, int ACT, int BK, int NB, bool PAIRED, bool SPLIT>
__global__ __launch_bounds__(SPLIT ? 512 : 256, BK == 32 ? 3 : 1) void gemm_mfma_kernel(const uint16_t *__restrict__ in,
                                                                        const uint16_t *__restrict__ weight,
                                                                        const uint16_t *__restrict__ bias,
                                                                        const uint16_t *residual, uint16_t *out, int N,
                                                                        int K, int tilesN, int tilesM) {
  using M = Mma<T>;
  using v8 = typename M::v8;
  using v4 = typename M::v4;
  static_assert((BK == 32 || BK == 64) && (NB == 4 || NB == 3) && (!PAIRED || BK == 32) && (!SPLIT || BK == 64),
                "tile geometry");
  constexpr int kBN = 32 * NB;
  constexpr int kSlice = 256 * BK;                   // bytes of an input slice, and of a weight slice at full pitch
  constexpr int kARow = BK * 2;                      // bytes per row of the input slice: 64 / 128
  constexpr int NC = BK / 16;                        // MFMA k-steps per reduction step: 2 / 4
  constexpr int NL = BK / 16 / (SPLIT ? 2 : 1);      // load instructions per wavefront and slice: 2 / 4 (2 when 8 wavefronts share them)
  constexpr int NCW = NC / (SPLIT ? 2 : 1);          // MFMA k-steps a wavefront takes per reduction step
  constexpr int CPR = BK / 8, RPI = 64 / CPR;        // input slice: chunks per row, rows per load instruction
  constexpr int WN = NB == 4 ? 2 : 1, WM = 4 / WN;   // wavefront grid over the tile: 2 x 2 or 4 x 1
  constexpr int MB = 4 / WM, NBW = NB / WN;          // 32 x 32 accumulators per wavefront: MB x NBW = 2 x 2 or 1 x 3
  constexpr int kOutStride = 32 * NBW + 4;           // staging row stride of a wavefront's part, in elements

  // Ring of kRing stages, each an input slice followed by a weight slice;
  // reused as the output staging area at the end.
  // PAIRED: two buffers of 16 KiB, each the input rows of two steps (128 rows of
  // 128 bytes), then two weight slices of 8 KiB.
  constexpr int kPairBytes = 16384, kWBase = 2 * kPairBytes;
  constexpr int kLds = PAIRED ? kWBase + 2 * 8192 : kRing * 2 * kSlice;
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kLds];
  static_assert(4 * 32 * MB * kOutStride * 2 <= kLds, "output staging must fit in the ring");

  // Tile order.  A contiguous run of work items goes to each of the 8 XCDs
  // (consecutive block ids are dealt round-robin to the XCDs), and consecutive
  // work items walk down kGroup rows of tiles before stepping one column, so
  // that the ~96 blocks resident on an XCD form a compact patch of tiles: the
  // slices they load per step are then few (8 input + 12 weight slices instead
  // of 2 + 64 for a row-major sweep of a wide matrix) and hit in that XCD's L2.
  constexpr int kGroup = 8;
  // (the grid is tilesM x tilesN blocks; both are explicit arguments - fourteen dwords in all,
  // what the command processor preloads into SGPRs - rather than gridDim, a kernarg-segment load)
  const int nblk = tilesM * tilesN;
  const int bid = blockIdx.x;
  const int wid = (nblk % 8 == 0) ? (bid % 8) * (nblk / 8) + bid / 8 : bid;
  const int perGroup = kGroup * tilesN;
  const int firstM = (wid / perGroup) * kGroup;
  const int groupRows = tilesM - firstM < kGroup ? tilesM - firstM : kGroup;
  const int inGroup = wid % perGroup;
  const int m0 = (firstM + inGroup % groupRows) * kBM;
  const int n0 = (inGroup / groupRows) * kBN;

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  // SPLIT: eight wavefronts; 0-3 and 4-7 cover the tile in the same way and take the
  // lower and the upper half of every reduction step, all eight share the loads.
  const int mover = __builtin_amdgcn_readfirstlane(tid / 64);
  const int khalf = SPLIT ? mover / 4 : 0;
  const int wave = SPLIT ? mover % 4 : mover;
  const int l32 = lane % 32;
  const int hl = lane / 32;
  const int wm = wave / WN, wn = wave % WN; // the wavefront's part of the tile

  // ---- slice movers: HBM -> LDS, 16 bytes per lane ----------------------------
  // One wavefront instruction fills 1 KiB: RPI rows of the input slice or 4 rows
  // of the weight slice; every wavefront moves a quarter of both.  In a 96-column
  // tile the lanes that would fetch the chunks beyond column 95 fetch a chunk of
  // the tile again instead: it lands in the unread tail of the 256-byte pitch.
  // (Masking those lanes off would put the load under divergent control flow,
  // where its scalar operands are no longer scalar to the compiler.)
  const char *abase = reinterpret_cast<const char *>(in) + (size_t)m0 * K * 2;
  const char *wbase = reinterpret_cast<const char *>(weight) + (size_t)n0 * 2;
  uint32_t aoff[NL], woff[NL];
#pragma unroll
  for (int i = 0; i < NL; i++) {
    const int arow = RPI * (NL * mover + i) + lane / CPR;
    aoff[i] = (uint32_t)arow * (uint32_t)K * 2u + (uint32_t)(((lane % CPR) ^ aSwz<BK>(arow)) * 16);
    const int wrow = 4 * (NL * mover + i) + lane / 16;
    int wchunk = (lane % 16) ^ wSwz(wrow);
    if (wchunk >= 4 * NB) wchunk -= 4;
    woff[i] = (uint32_t)wrow * (uint32_t)N * 2u + (uint32_t)(wchunk * 16);
  }
  // PAIRED: the input rows of two steps at once, 8 rows of 128 bytes per load
  // instruction, four instructions per wavefront.
  uint32_t aoffP[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int arow = 8 * (4 * wave + i) + lane / 8;
    aoffP[i] = (uint32_t)arow * (uint32_t)K * 2u + (uint32_t)(((lane % 8) ^ aSwz<64>(arow)) * 16);
  }
  // Inline assembly keeps these loads out of the compiler's wait-count
  // bookkeeping, which would otherwise wait for every load in flight before
  // any later LDS read; completion is tracked by hand (2 * NL loads per stage
  // and wavefront).
  const uint32_t ldsBase = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) unsigned char *)smem);
  // M0 is on the clobber list so that the statement counts as a definition of it
  // (the compiler reserves M0 and notes that such a clobber is not saved and restored:
  // nothing here needs it preserved).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  auto dma16 = [&](uint32_t voffset, const char *sbase, uint32_t ldsAddr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voffset), "s"(sbase), "s"(ldsAddr)
                 : "memory", "m0");
  };
#pragma clang diagnostic pop
  auto issueStage = [&](int kt) {
    const uint32_t adst = ldsBase + (uint32_t)((kt % kRing) * (2 * kSlice) + (NL * mover) * 1024);
    const uint32_t wdst = adst + kSlice;
    const char *ag = abase + (size_t)kt * kARow;
    const char *wg = wbase + (size_t)kt * BK * N * 2;
#pragma unroll
    for (int i = 0; i < NL; i++) {
      dma16(aoff[i], ag, adst + i * 1024);
      dma16(woff[i], wg, wdst + i * 1024);
    }
  };

  auto issueWeights = [&](int kt) { // PAIRED: the weight slice of step kt
    const uint32_t wdst = ldsBase + (uint32_t)(kWBase + (kt % 2) * 8192 + (2 * wave) * 1024);
    const char *wg = wbase + (size_t)kt * 32 * N * 2;
#pragma unroll
    for (int i = 0; i < 2; i++) dma16(woff[i], wg, wdst + i * 1024);
  };
  auto issuePair = [&](int p) { // PAIRED: the input rows of steps 2p and 2p + 1
    const uint32_t adst = ldsBase + (uint32_t)((p % 2) * kPairBytes + (4 * wave) * 1024);
    const char *ag = abase + (size_t)p * 128;
#pragma unroll
    for (int i = 0; i < 4; i++) dma16(aoffP[i], ag, adst + i * 1024);
  };

  const int nk = K / BK;
  if (PAIRED) {
    issueWeights(0);
    issuePair(0);
  } else {
#pragma unroll
    for (int t = 0; t < kRing - 1; t++)
      if (t < nk) issueStage(t);
  }

  // ---- operand addresses inside a stage ---------------------------------------
  // in^T: lane (row 32*MB*wm + 32mb + l32, k chunk 2c + hl) reads 16 bytes.
  uint32_t afrag[MB][NC];
#pragma unroll
  for (int mb = 0; mb < MB; mb++)
#pragma unroll
    for (int c = 0; c < NC; c++) {
      const int row = wm * (32 * MB) + 32 * mb + l32;
      afrag[mb][c] = (uint32_t)(row * kARow + (((2 * c + hl) ^ aSwz<BK>(row)) * 16));
    }
  // W^T: as a source of the transposing read, lane L of a 16-lane group g points
  // at k row 8*hl + L/4 (+ 16c, + 4 for the upper k-slots) and the four columns
  // n = 32nb + 16*(g%2) + 4*(L%4) .. +3.
  // PAIRED: row of a 128-byte pitch, k chunk 4 * (kt % 2) + 2c + hl of the pair's 8;
  // the step's half is bit 2 of the chunk, i.e. bit 6 of the address, and passes
  // through the XOR swizzle unchanged.
  uint32_t afragP[MB][2];
#pragma unroll
  for (int mb = 0; mb < MB; mb++)
#pragma unroll
    for (int c = 0; c < 2; c++) {
      const int row = wm * (32 * MB) + 32 * mb + l32;
      afragP[mb][c] = (uint32_t)(row * 128 + (((2 * c + hl) ^ aSwz<64>(row)) * 16));
    }
  uint32_t wfrag[NBW]; // relative to the weight slice
  {
    const int g = lane / 16, L = lane % 16, r = L % 4, j = L / 4;
#pragma unroll
    for (int nb = 0; nb < NBW; nb++) {
      const int chunk = (4 * (NBW * wn + nb) + 2 * (g % 2) + r / 2) ^ wSwz(j);
      wfrag[nb] = (uint32_t)((8 * hl + j) * kWRow + chunk * 16 + 8 * (r % 2));
    }
  }

  f32x16 acc[NBW][MB]; // [nb][mb]: rows n, columns m
#pragma unroll
  for (int nb = 0; nb < NBW; nb++)
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[nb][mb][i] = 0.0f;

  for (int kt = 0; kt < nk; kt++) {
    uint32_t aBase, wBase; // LDS addresses of this step's input rows and weight slice
    if (PAIRED) {
      // Issue order is: weights of step 1, pair 1, weights of step 2, weights of
      // step 3, pair 2, ...  An even step needs its pair (issued two steps ago)
      // and its weights (issued one step ago): everything in flight.  An odd step
      // needs its weights only, issued just before the next pair: 4 loads may fly.
      if ((kt & 1) == 0 || kt + 1 >= nk) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      __syncthreads();
      if (kt + 1 < nk) issueWeights(kt + 1);
      if ((kt & 1) == 0 && kt + 2 < nk) issuePair(kt / 2 + 1);
      aBase = ldsBase + (uint32_t)(((kt / 2) % 2) * kPairBytes);
      wBase = ldsBase + (uint32_t)(kWBase + (kt % 2) * 8192);
    } else {
      // The loads of stage kt (and of nothing later) must have landed; the barrier
      // makes every wavefront's share visible and says that everybody is done
      // with stage kt-1, which the next load overwrites.
      if (kt + 1 < nk) {
        if (NL == 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      __syncthreads();
      if (kt + kRing - 1 < nk) issueStage(kt + kRing - 1);
      aBase = ldsBase + (uint32_t)((kt % kRing) * (2 * kSlice));
      wBase = aBase + kSlice;
    }

    if (SPLIT) wBase += (uint32_t)khalf * (16 * NCW * kWRow); // this half's k-steps: 32 rows further down the weight slice
#pragma unroll
    for (int c = 0; c < NCW; c++) {
      v8 b[MB], a[NBW];
#pragma unroll
      for (int mb = 0; mb < MB; mb++) {
        // SPLIT: the upper half's k-steps are chunk bit 2 of the input rows, which passes through the swizzle
        const uint32_t off = PAIRED ? (afragP[mb][c & 1] ^ ((uint32_t)(kt & 1) << 6))
                                    : SPLIT ? (afrag[mb][c] ^ ((uint32_t)khalf << 6)) : afrag[mb][c];
        b[mb] = *reinterpret_cast<const v8 __attribute__((address_space(3))) *>((const lds_u8 *)(uintptr_t)(aBase + off));
      }
#pragma unroll
      for (int nb = 0; nb < NBW; nb++) {
        const lds_u8 *p = (const lds_u8 *)(uintptr_t)(wBase + wfrag[nb]) + 16 * c * kWRow;
        const v4 lo = M::readTr(p);             // k-slots 0..3
        const v4 hi = M::readTr(p + 4 * kWRow); // k-slots 4..7
        a[nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
#pragma unroll
      for (int nb = 0; nb < NBW; nb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++) acc[nb][mb] = M::run(a[nb], b[mb], acc[nb][mb]);
    }
  }

  // ---- epilogue: bias, activation, residual; transpose through LDS; store ------
  __syncthreads(); // every wavefront is done reading the slices
  if (SPLIT) {
    // the upper half hands its accumulators to the lower half through LDS: 16
    // bytes per lane and register group, consecutive lanes consecutive
    float4v *red = reinterpret_cast<float4v *>(smem) + wave * (NBW * MB * 4 * 64);
    if (khalf == 1) {
#pragma unroll
      for (int nb = 0; nb < NBW; nb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
          for (int g = 0; g < 4; g++)
            red[((nb * MB + mb) * 4 + g) * 64 + lane] = float4v{acc[nb][mb][4 * g], acc[nb][mb][4 * g + 1],
                                                               acc[nb][mb][4 * g + 2], acc[nb][mb][4 * g + 3]};
    }
    __syncthreads();
    if (khalf == 0) {
#pragma unroll
      for (int nb = 0; nb < NBW; nb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            const float4v other = red[((nb * MB + mb) * 4 + g) * 64 + lane];
            acc[nb][mb][4 * g] += other[0];
            acc[nb][mb][4 * g + 1] += other[1];
            acc[nb][mb][4 * g + 2] += other[2];
            acc[nb][mb][4 * g + 3] += other[3];
          }
    }
    __syncthreads(); // the staging area below overlaps what the other wavefronts have just read
    if (khalf == 1) return;
  }
  uint16_t *stage = reinterpret_cast<uint16_t *>(smem) + wave * (32 * MB * kOutStride);
  const int mw = m0 + wm * (32 * MB), nw = n0 + wn * (32 * NBW); // origin of the wavefront's part
  // All bias pieces of the part first, then per 32-column block all of its
  // residual pieces, so that the loads of a batch are in flight together.
  v4 braw[NBW][4];
#pragma unroll
  for (int nb = 0; nb < NBW; nb++)
#pragma unroll
    for (int g = 0; g < 4; g++)
#pragma unroll
      for (int i = 0; i < 4; i++) braw[nb][g][i] = M::narrow(0.0f);
  if (bias) {
#pragma unroll
    for (int nb = 0; nb < NBW; nb++)
#pragma unroll
      for (int g = 0; g < 4; g++) braw[nb][g] = *reinterpret_cast<const v4 *>(bias + nw + 32 * nb + 8 * g + 4 * hl);
  }
#pragma unroll
  for (int nb = 0; nb < NBW; nb++) {
    v4 rraw[4][MB];
#pragma unroll
    for (int g = 0; g < 4; g++)
#pragma unroll
      for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int i = 0; i < 4; i++) rraw[g][mb][i] = M::narrow(0.0f);
    if (residual) {
#pragma unroll
      for (int g = 0; g < 4; g++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
          rraw[g][mb] = *reinterpret_cast<const v4 *>(residual + (size_t)(mw + 32 * mb + l32) * N + nw + 32 * nb +
                                                      8 * g + 4 * hl);
    }
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const int nloc = 32 * nb + 8 * g + 4 * hl; // four consecutive columns of the part
#pragma unroll
      for (int mb = 0; mb < MB; mb++) {
        const int mloc = 32 * mb + l32;
        float x[4];
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = acc[nb][mb][4 * g + i] + M::widen(braw[nb][g][i]);
        if (ACT == ACT_RELU) {
#pragma unroll
          for (int i = 0; i < 4; i++) x[i] = x[i] > 0.0f ? x[i] : 0.0f;
        } else if (ACT == ACT_GELU) {
#pragma unroll
          for (int i = 0; i < 4; i++) x[i] = gelu_erfc(x[i]);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] += M::widen(rraw[g][mb][i]);
        v4 o;
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = M::narrow(x[i]);
        *reinterpret_cast<v4 *>(&stage[mloc * kOutStride + nloc]) = o;
      }
    }
  }
  // Each wavefront reads back only what it wrote: no block barrier needed, the
  // LDS accesses of one wavefront are ordered.
  constexpr int kOutChunks = 4 * NBW; // 16-byte chunks per row of the part
#pragma unroll
  for (int it = 0; it < 32 * MB * kOutChunks / 64; it++) {
    const int chunk = it * 64 + lane;
    const int r = chunk / kOutChunks, cidx = chunk % kOutChunks;
    // 8-byte LDS reads: the staging stride is 8-byte but not 16-byte aligned
    const u32x2 lo = *reinterpret_cast<const u32x2 *>(&stage[r * kOutStride + cidx * 8]);
    const u32x2 hi = *reinterpret_cast<const u32x2 *>(&stage[r * kOutStride + cidx * 8 + 4]);
    const u32x4 val = {lo[0], lo[1], hi[0], hi[1]};
    *reinterpret_cast<u32x4 *>(out + (size_t)(mw + r) * N + nw + cidx * 8) = val;
  }
}

template <typename T, int BK, int NB, bool PAIRED, bool SPLIT = false>
void launchTile(const uint16_t *a, const uint16_t *w, const uint16_t *b, const uint16_t *r, uint16_t *o, int64_t M,
                int64_t N, int64_t K, int act, hipStream_t stream) {
  const int tilesN = (int)(N / (32 * NB));
  const dim3 grid((unsigned)((M / kBM) * tilesN)), block(SPLIT ? 512 : 256);
  if (act == ACT_GELU)
    gemm_mfma_kernel<T, ACT_GELU, BK, NB, PAIRED, SPLIT><<<grid, block, 0, stream>>>(a, w, b, r, o, (int)N, (int)K, tilesN, (int)(M / kBM));
  else if (act == ACT_RELU)
    gemm_mfma_kernel<T, ACT_RELU, BK, NB, PAIRED, SPLIT><<<grid, block, 0, stream>>>(a, w, b, r, o, (int)N, (int)K, tilesN, (int)(M / kBM));
  else
    gemm_mfma_kernel<T, ACT_NONE, BK, NB, PAIRED, SPLIT><<<grid, block, 0, stream>>>(a, w, b, r, o, (int)N, (int)K, tilesN, (int)(M / kBM));
}

// Tile width: the one under which the busiest CU carries the fewest columns
// (tiles are dealt evenly, so that CU holds ceil(tiles / CUs) of them); 128 on
// a tie.  Reduction step: 64 when no CU gets a second tile; otherwise 32, with
// the input rows fetched in pairs of steps when K allows.
template <typename T>
void launch(const void *in, const void *weight, const void *bias, const void *residual, void *out, int64_t M,
            int64_t N, int64_t K, int act, hipStream_t stream) {
  const int64_t cus = numComputeUnits();
  auto load = [&](int64_t width) -> int64_t {
    if (N % width) return INT64_MAX;
    const int64_t tiles = (M / kBM) * (N / width);
    return (tiles + cus - 1) / cus * width;
  };
  const bool narrow = load(96) < load(128);
  const int64_t tiles = (M / kBM) * (N / (narrow ? 96 : 128));
  const bool deep = tiles <= cus && K % 64 == 0;
  const auto *a = static_cast<const uint16_t *>(in);
  const auto *w = static_cast<const uint16_t *>(weight);
  const auto *b = static_cast<const uint16_t *>(bias);
  const auto *r = static_cast<const uint16_t *>(residual);
  auto *o = static_cast<uint16_t *>(out);
  const bool paired = !deep && K % 64 == 0;
  if (narrow) {
    if (deep) launchTile<T, 64, 3, false, true>(a, w, b, r, o, M, N, K, act, stream);
    else if (paired) launchTile<T, 32, 3, true>(a, w, b, r, o, M, N, K, act, stream);
    else launchTile<T, 32, 3, false>(a, w, b, r, o, M, N, K, act, stream);
  } else {
    if (deep) launchTile<T, 64, 4, false, true>(a, w, b, r, o, M, N, K, act, stream);
    else if (paired) launchTile<T, 32, 4, true>(a, w, b, r, o, M, N, K, act, stream);
    else launchTile<T, 32, 4, false>(a, w, b, r, o, M, N, K, act, stream);
  }
  MGPU_CHECK_LAUNCH("gemm_mfma_kernel");
}

} // namespace

bool gemmMfmaSupports(DType dt, const void *in, const void *weight, const void *bias, const void *residual,
                      const void *out, int64_t M, int64_t N, int64_t K) {
  if (dt != DType::F16 && dt != DType::BF16) return false;
  if (M <= 0 || N <= 0 || K <= 0 || M % kBM || (N % 128 && N % 96) || K % 32) return false;
  // 32-bit lane offsets inside a slice, 31-bit tile counts
  if (K > (1 << 20) || N > (1 << 20) || (M / kBM) * (N / 96) > 0x7fffffffLL) return false;
  if (!aligned16(in) || !aligned16(weight) || !aligned16(out)) return false;
  if (bias && (reinterpret_cast<uintptr_t>(bias) & 7u)) return false;
  if (residual && !aligned16(residual)) return false;
  return true;
}

void gemmMfma(DType dt, const void *in, const void *weight, const void *bias, const void *residual, void *out,
              int64_t M, int64_t N, int64_t K, int act, hipStream_t stream) {
  if (!gemmMfmaSupports(dt, in, weight, bias, residual, out, M, N, K))
    fail("gemmMfma: shape, type or alignment not supported by the hand-written kernel");
  if (act != ACT_NONE && residual) fail("gemmMfma: an activation cannot be combined with a residual");
  if (dt == DType::F16)
    launch<_Float16>(in, weight, bias, residual, out, M, N, K, act, stream);
  else
    launch<bf16_t>(in, weight, bias, residual, out, M, N, K, act, stream);
}

} // namespace mgpu
