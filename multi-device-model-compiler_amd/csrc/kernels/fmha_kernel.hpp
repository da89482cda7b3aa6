// The fused multi-head attention forward kernel for gfx950 MFMA (the launcher is fmha.hip): tile geometries for head_dim 64,
// 128 and 256, every other multiple of 8 up to 256 inside the next larger one.
//
// Replaces the cubin kernels the reference dispatches through
// FusedMHARunnerFP16v2 (3rdparty/trt_fused_multihead_attention/
// qkvToContext.cu:162-199,306-315; fused_multihead_attention_v2.h:5278-5377)
// at lib/Kernels/GPU/LLM.cu:79-81: O = softmax(scale * Q K^T + mask) V on packed
// [B,S,3,H,D] QKV, output [B,S,H*D].  One kernel family for every S: flash
// style, no score matrix in memory.
//
// Work decomposition.  A 256-thread block (4 wavefronts) owns BM = 128 * NQ
// consecutive queries of one (batch, head); each wavefront owns NQ blocks of 32
// queries.  Key/value tiles of 8 KiB (64 keys at head_dim 64; 16 KiB at 128 and
// 256, see Geo below; the comments give the head_dim 64 numbers) travel HBM ->
// LDS directly (global_load_lds, 16 bytes per lane, no register staging) into a
// ring of three LDS stages shared by the 4 wavefronts, so two tiles are always
// in flight behind the one being consumed.
//
// MFMA formulation (v_mfma_f32_32x32x16_{f16,bf16}; operand lane layout: lane l
// supplies row/col l%32 and k-slots 8*(l/32)..+7; the 32x32 accumulator gives
// lane l column l%32 and rows 8*(i/4) + 4*(l/32) + i%4 for register i):
//   S^T[key, query] = K[key, :] . Q[query, :]      A = K tile (LDS), B = Q (registers)
//   O^T[d,   query] = V^T[d, key] . P^T[key, query] A = V^T tile (LDS), B = P (registers)
// Computing the transposed products puts one query per lane column, so
//   * a softmax row is 16 accumulator registers in each of two lanes (l, l^32):
//     the row maximum and sum need in-lane work plus ONE lane exchange;
//   * the S^T accumulators ARE the B operand of the second product: registers
//     8m..8m+7 of a lane hold keys {16m + 4*(l/32) + 0..3, 16m + 8 + 4*(l/32) + 0..3}
//     and the contraction over keys does not care in which k-slot a key sits as
//     long as the A operand (V^T) is read with the same assignment - two 8-byte
//     LDS reads per operand.  P never leaves registers.
// Both tiles sit in LDS row-major as in memory (64 rows of 128 bytes).  The
// direct loads write 1 KiB of consecutive LDS per wavefront instruction, so
// rows cannot be padded; instead each lane fetches the 16-byte chunk
// c ^ swizzle(row) of its row, which makes the K operand reads (ds_read_b128,
// 16 rows per cycle) and the V operand reads conflict free.  V^T operands come
// from ds_read_b64_tr_b16, the transposing LDS read of gfx950: within 16
// lanes, lane L receives element L%4 of the four 8-byte rows addressed by
// lanes L/4, L/4+4, L/4+8, L/4+12 - four keys of one d column.
//
// Softmax runs in fp32 in base 2: p = exp2(s*c - m*c), c = scale*log2(e), the
// scale staying in fp32.  At head_dim 64 one score pays for only 256 MFMA
// flops, i.e. 16 issue cycles per wavefront, and a wavefront issues in order:
// VALU work is free only while it sits between MFMAs whose results it does not
// need.  So the per-score work is trimmed to one fma, one exp2, half a convert
// and one add, and the row maximum is taken out of the hot path entirely:
//   * m is a stale reference, not the running maximum, and starts at 0.  P is
//     produced optimistically against it; fp16 holds p up to 2^16 with the
//     same relative precision everywhere above 2^-14, so any reference within
//     about +-12 (base-2 units) of the true row maximum is as good as the
//     maximum itself.  A reference that is too low shows up as a tile row sum
//     beyond 2^15, an initial one that is too high as a first sum below 2^-6.  Only
//     then does the wavefront take the slow path: true row maximum, rescale of
//     O and l (or a restart, if nothing has been accumulated yet), P
//     recomputed.  O / l does not depend on which m was used.  Ordinary
//     logits (|s * scale| up to ~8) never leave the fast path, whose softmax
//     is a single pass of fma / exp2 / add / convert over the scores;
//   * the row sum is a plain fp32 add per score.  v_dot2_f32_f16 over the
//     converted P pairs would halve the instruction count, but it runs on the
//     matrix pipeline: measured between MFMAs it costs 6 cycles that do not
//     overlap, where add, fma, max3 and the f16 converts overlap completely
//     and v_exp_f32 costs about 2;
//   * accumulators stay in VGPRs (no AGPR copies);
//   * three wavefronts share a SIMD (145 VGPRs) and are left to drift apart, so
//     that one is in an MFMA phase while another does its softmax; s_setprio
//     lets the MFMA phases win the issue slot.
// The output tile is transposed through LDS so that every store instruction
// writes whole 128-byte rows.
#pragma once
#include "common.hpp"
#include "types.hpp"
#include "mfma.hpp"

namespace mgpu {

namespace fmha_detail {

// Geometry per head dimension D (64, 128 or 256).  At D = 64 a K or V tile is 8 KiB
// (64 keys of 128 bytes, 8 MFMAs for the scores and 8 for P.V), the ring has three
// stages and three blocks share a CU (145 VGPRs, three wavefronts per SIMD).  At
// D = 128 and 256 a tile is 16 KiB (64 keys of 256 bytes or 32 of 512: 16 + 16 MFMAs
// per tile, half as many barriers and bursts of tile loads per MFMA) and the ring has
// two stages, so that two blocks share a CU's LDS; accumulators and Q operands (64 + 32
// registers at 128, 128 + 64 at 256) leave room for two wavefronts per SIMD either way.
// (D = 128 with 8 KiB tiles of 32 keys, a ring of three and three wavefronts per SIMD at
// the 168-register limit measured 5-12 % slower from S = 128 to S = 8192 - b32 s512 h8
// 50 against 44-51 us, b1 s8192 h8 273 against 257 - and 2 % faster only on the largest
// grid tried, b4 s2048 h32.)
template <int D> struct Geo {
  static_assert(D == 64 || D == 128 || D == 256, "head dimension 64, 128 or 256");
  static constexpr int kTileBytes = D >= 128 ? 16384 : 8192; // one K or V tile, unpadded rows
  static constexpr int kStages = D >= 128 ? 2 : 3;           // LDS ring depth
  static constexpr int kStageBytes = 2 * kTileBytes;         // a stage: the K tile followed by the V tile
  static constexpr int LPW = kTileBytes / 4096;     // 1 KiB load instructions per wavefront and tile half: 2 / 4 / 4
  static constexpr int kBN = kTileBytes / (D * 2);  // keys per tile: 64 / 64 / 32
  static constexpr int KB = kBN / 32;               // 32-key score blocks per tile: 2 / 2 / 1
  static constexpr int DC = D / 16;                 // MFMA k-steps over the head dimension: 4 / 8 / 16
  static constexpr int DB = D / 32;                 // 32-row blocks of O^T: 2 / 4 / 8
  static constexpr int rowBytes = D * 2;            // 128 / 256 / 512
  static constexpr int CPR = rowBytes / 16;         // 16-byte chunks per row: 8 / 16 / 32
  static constexpr int RPI = 64 / CPR;              // tile rows one wavefront load instruction fills: 8 / 4 / 2
  static constexpr int OS = D + 4;                  // output staging row stride in elements
  // The swizzles below act on the low four bits of a row's chunk index, so operand
  // addresses 16 chunks (256 bytes) apart differ by a constant: only KF distinct K
  // operand addresses and VF distinct V operand addresses are kept in registers.
  static constexpr int KF = DC < 8 ? DC : 8;
  static constexpr int VF = DB < 4 ? DB : 4;
  // chunk swizzles (XOR on the 16-byte chunk index of a row) that keep the K
  // operand reads and the transposing V reads free of bank conflicts
  __host__ __device__ static constexpr int kSwz(int row) { return D == 64 ? ((row >> 1) & 7) : (row & 15); }
  __host__ __device__ static constexpr int vSwz(int row) { return D == 64 ? (((row >> 1) & 1) << 2) : ((row & 3) << 2); }
};
// A lane's share of a tile's row sum above kSumLimit (or NaN) sends the
// wavefront to the repair path: any p beyond the fp16 range (65504) pushes the
// fp32 sum past it, and a legitimate sum that large only costs one needless
// repair.  A sum below kSumFloor on the first tile means the initial reference
// sits so far above the scores that P is leaving fp16's normal range (the
// largest p of a row is at least sum / keys): the reference is then lowered to
// the tile's maximum.  Every query sees a key in the first tile (key 0 is
// valid under both masks), so from then on its running sum stays above the
// floor - a raised reference comes with a tile whose largest p is 1 - and the
// test is not needed again.
constexpr float kSumLimit = 32768.0f;
constexpr float kSumFloor = 0.015625f;

// TRACE (the profiling entry point only): wavefront 0 of every block records
// the shader clock at entry, when its first tile has landed, after its last
// tile and after its stores, the device-wide constant clock at entry and
// exit, and the shader clocks its tiles spent waiting for the tile to land
// (wait + barrier), in the score MFMAs, in the softmax and in the P.V MFMAs:
// ten uint64 per block in `stamps`.
//
// PAD: the head dimension in memory, dHead (a multiple of 8 below D), is smaller
// than the tile geometry D the kernel computes in.  Rows in memory are dHead
// elements long; a lane whose 16-byte chunk of a K or V row lies beyond dHead
// fetches chunk 0 of that row instead (in bounds, finite wherever the row is),
// Q is zero there, so the scores do not see the K filler, and the O^T rows the V
// filler feeds are never stored.
template <typename T, int D, int NQ, bool CAUSAL, bool TRACE = false, bool PAD = false>
__global__ __launch_bounds__(256, (CAUSAL && D == 64) ? 3 : 2) void fmha_fwd_kernel(const uint16_t *__restrict__ qkv,
                                                              const int32_t *__restrict__ seqlens,
                                                              const int32_t *__restrict__ cuSeqlens,
                                                              uint16_t *__restrict__ out, int S, int H,
                                                              int nQB, float scale_log2e, int pairItems,
                                                              int nblk, int dHead,
                                                              uint64_t *__restrict__ stamps) {
  // (nblk is the grid size: as an explicit argument it is one of the fourteen dwords the
  // command processor preloads into SGPRs; gridDim would be a load from the kernarg segment)
  uint64_t tEntry = 0, wEntry = 0, tFirstTile = 0, tLoopEnd = 0;
  uint64_t cWait = 0, cScores = 0, cSoftmax = 0, cPV = 0, tMark = 0;
  if (TRACE) {
    tEntry = clock64();
    wEntry = wall_clock64();
  }
  using M = Mma<T>;
  using v8 = typename M::v8;
  using v4 = typename M::v4;
  using G = Geo<D>;
  constexpr int BM = 128 * NQ;
  constexpr int kBN = G::kBN;
  constexpr int kStages = G::kStages, kTileBytes = G::kTileBytes, kStageBytes = G::kStageBytes, LPW = G::LPW;
  const int kD = PAD ? dHead : D;           // elements per head in memory
  const int validChunks = PAD ? dHead / 8 : G::CPR; // 16-byte chunks of a row that exist

  // Ring of kStages stages, each a K tile followed by a V tile; reused as the
  // output staging area at the end (at D = 256 the staging rows, padded against
  // bank conflicts, need 1 KiB more than the ring).
  constexpr int kRingBytes = kStages * kStageBytes;
  constexpr int kStagingBytes = 4 * NQ * 32 * G::OS * 2;
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kRingBytes > kStagingBytes ? kRingBytes : kStagingBytes];

  // Work-item order: query blocks of one (batch, head) are consecutive, and a
  // contiguous run of work items goes to each of the 8 XCDs (consecutive block
  // ids are dealt round-robin to the XCDs), so the blocks that re-read the
  // same K/V share one L2.
  const int bid = blockIdx.x;
  const int wid = (nblk % 8 == 0) ? (bid % 8) * (nblk / 8) + bid / 8 : bid;
  // Causal: query block i of a (batch, head) needs i + 1 of the nQB key
  // ranges.  When the launcher asks for it (pairItems), block i and block
  // nQB - 1 - i are given to one work item, so that every work item carries the
  // same number of tiles; left alone, the items with the last query blocks run
  // as long as without the mask while the others sit idle.  At head_dim 64 the
  // short block goes first, so that the long one starts with the K/V tiles the
  // short one has just read (b32 s512 h12: 29.0 -> 27.6 us); at 128, with its ring
  // of two stages, the long block first measured faster (b8 s1024 h16: 46.5
  // against 49.6 us).
  constexpr bool kCanPair = CAUSAL && D <= 128; // at 256 the second pass is compiled out
  const bool paired = kCanPair && pairItems == 1;
  const int nItems = paired ? (nQB + 1) / 2 : nQB; // work items per (batch, head)
  int item = wid % nItems;
  int bh = wid / nItems;
  // Unpaired causal launches carry blocks of nQB different lengths.  pairItems = 2 asks for them
  // longest first within each XCD's run: the long blocks start at once and the short ones fill in
  // behind them, where index order gave a compute unit two blocks of the same length - two of the
  // longest for a quarter of the units (b8 s512 h16 d128: 23.0 -> 20.7 us, b16 s512 h12 d64: 19.5 ->
  // 14.8 us, b2 s2048 h16 d64: 41.8 -> 34.6 us).
  if (CAUSAL && !paired && pairItems == 2 && nblk % 8 == 0 && (nblk / 8) % nQB == 0) {
    const int nbh = nblk / 8 / nQB; // (batch, head)s of this XCD
    const int rank = bid / 8;       // position in the XCD's dispatch order; 0 gets a longest block
    item = nQB - 1 - rank / nbh;
    bh = (bid % 8) * nbh + rank % nbh;
  } else if (CAUSAL && !paired && pairItems == 2) {
    // (batch, head)s that do not divide over the XCDs: longest first over the whole grid
    const int nbh = nblk / nQB;
    item = nQB - 1 - bid / nbh;
    bh = bid % nbh;
  }
  // Sequences of unequal length: a contiguous run of (batch, head)s per XCD is a few whole
  // sequences per XCD (one, at b8 h16), and the XCD that drew the longest sets the launch's
  // time.  Dealing the (batch, head)s round-robin instead gives every XCD some heads of every
  // sequence; the query blocks of one (batch, head) still share an XCD (b8 s512 h16 d128, key
  // counts 256..512: 23.0 -> 20.6 us; b64 s512 h12 d64, 1..512: 53.5 -> 49.3).  Not with one query
  // block per (batch, head): there the finer interleave of the rows over the XCDs costs more
  // than the balance gains (b32 s128 h12: 6.36 -> 6.53 us).
  if ((seqlens || cuSeqlens) && nQB >= 2 && nblk % 8 == 0 && (nblk / nItems) % 8 == 0 &&
      !(CAUSAL && !paired && pairItems == 2 && (nblk / 8) % nQB != 0)) {
    const int perXcd = nblk / nItems / 8;
    bh = (bh % perXcd) * 8 + bh / perXcd;
  }
  const int h = bh % H;
  const int b = bh / H;

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int l32 = lane % 32;
  const int hl = lane / 32;

  // (The loop over the two blocks of a pair starts here, ahead of the sequence
  // bounds and the base addresses: recomputed per block they cost a few scalar
  // instructions, kept across the loop they cost registers the causal kernel
  // does not have - it spilled eight with the loop further down.)
  const int nParts = (kCanPair && paired && item != nQB - 1 - item) ? 2 : 1;
  auto runPart = [&](const int part) {
  // Two ways to say how long a sequence is.  seqlens: every sequence owns S
  // token rows, keys beyond seqlens[b] are masked, all S query rows are
  // produced.  cuSeqlens (b + 1 prefix sums, the reference's form): the token
  // rows are packed back to back, sequence b owns rows cuSeqlens[b] ..
  // cuSeqlens[b + 1] - 1 and no others exist for it; S bounds its length.
  int kvlen = S, rows = S; // admissible keys; token rows that exist
  size_t tok0 = (size_t)b * S;
  if (cuSeqlens) {
    const int first = cuSeqlens[b];
    kvlen = cuSeqlens[b + 1] - first;
    kvlen = kvlen < 0 ? 0 : (kvlen > S ? S : kvlen);
    rows = kvlen;
    tok0 = (size_t)first;
    // Nothing to do for an empty sequence, or for a block all of whose queries lie
    // beyond the sequence (a paired work item always holds an early block).
    if (rows == 0 || (!paired && item * BM >= rows)) return;
  } else if (seqlens) {
    kvlen = seqlens[b];
    kvlen = kvlen < 0 ? 0 : (kvlen > S ? S : kvlen);
  }
  const uint32_t tokBytes = (uint32_t)3 * H * kD * 2; // bytes per token row
  const char *qbase = reinterpret_cast<const char *>(qkv) + (tok0 * 3 * H + h) * kD * 2;
  const char *kbase = qbase + (size_t)H * kD * 2;
  const char *vbase = qbase + (size_t)2 * H * kD * 2;

  constexpr bool kShortFirst = D == 64;
  const int qb = paired ? ((part == 0) == kShortFirst ? item : nQB - 1 - item) : item;
  const int q0 = qb * BM + wave * (NQ * 32); // first query of this wavefront
  int kend = kvlen;
  if (CAUSAL) {
    int lastq = qb * BM + BM - 1;
    lastq = lastq < S - 1 ? lastq : S - 1;
    kend = kend < lastq + 1 ? kend : lastq + 1;
  }
  const int nkt = (kend + kBN - 1) / kBN;

  // ---- tile movers: HBM -> LDS, 16 bytes per lane ---------------------------
  // One wavefront instruction fills 1 KiB = RPI tile rows; wavefront w moves
  // a quarter (LPW KiB) of both tiles.  Lane l lands in LDS chunk l % CPR of row
  // l / CPR and fetches global chunk (l % CPR) ^ swizzle(row).
  const int mrow = lane / G::CPR, mchunk = lane % G::CPR;
  auto srcChunk = [&](int chunk) { return (PAD && chunk >= validChunks) ? 0 : chunk; };
  // Offsets of this lane's loads inside a tile.  Where registers are short (D = 256)
  // they are recomputed at every use from the lane's row and chunk - the copy that
  // goes through the empty asm statement keeps the compiler from hoisting the
  // arithmetic out of the tile loop and spilling its results instead.
  constexpr bool kRecomputeOffsets = D == 256;
  auto tileOffset = [&](int i, bool isV) {
    int mr = mrow;
    if (kRecomputeOffsets) asm volatile("" : "+v"(mr));
    const int row = G::RPI * (LPW * wave + i) + mr;
    return (uint32_t)row * tokBytes + (uint32_t)(srcChunk(mchunk ^ (isV ? G::vSwz(row) : G::kSwz(row))) * 16);
  };
  uint32_t koff[LPW], voff[LPW];
#pragma unroll
  for (int i = 0; i < LPW; i++) {
    koff[i] = kRecomputeOffsets ? 0u : tileOffset(i, false);
    voff[i] = kRecomputeOffsets ? 0u : tileOffset(i, true);
  }
  // The loads are written as inline assembly so that the compiler's wait-count
  // bookkeeping does not see them: it would otherwise wait for every load in
  // flight, prefetches included, before any later LDS read.  Completion is
  // tracked by hand with s_waitcnt vmcnt(n) below (2 * LPW loads per tile and wave).
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
  auto issueTile = [&](int kt) {
    const uint32_t kdst = ldsBase + (uint32_t)((kt % kStages) * kStageBytes + (LPW * wave) * 1024);
    const uint32_t vdst = kdst + kTileBytes;
    if (kt * kBN + kBN <= rows) { // whole tile inside the sequence
      const char *kg = kbase + (size_t)kt * kBN * tokBytes;
      const char *vg = vbase + (size_t)kt * kBN * tokBytes;
#pragma unroll
      for (int i = 0; i < LPW; i++) {
        dma16(kRecomputeOffsets ? tileOffset(i, false) : koff[i], kg, kdst + i * 1024);
        dma16(kRecomputeOffsets ? tileOffset(i, true) : voff[i], vg, vdst + i * 1024);
      }
    } else { // last tile of a ragged sequence: clamp the row, the mask hides it
#pragma unroll
      for (int i = 0; i < LPW; i++) {
        const int row = G::RPI * (LPW * wave + i) + mrow;
        int key = kt * kBN + row;
        key = key < rows ? key : rows - 1;
        const uint32_t rowOff = (uint32_t)key * tokBytes;
        dma16(rowOff + srcChunk(mchunk ^ G::kSwz(row)) * 16, kbase, kdst + i * 1024);
        dma16(rowOff + srcChunk(mchunk ^ G::vSwz(row)) * 16, vbase, vdst + i * 1024);
      }
    }
  };

  // Start the ring before anything else so the first tiles overlap the Q setup.
#pragma unroll
  for (int t = 0; t < kStages - 1; t++)
    if (t < nkt) issueTile(t);

  // Q as the B operand: lane (query l32, k-slots = d 16c + 8hl .. +7).
  v8 qf[NQ][G::DC];
#pragma unroll
  for (int qi = 0; qi < NQ; qi++) {
    int row = q0 + qi * 32 + l32;
    row = row < rows ? row : rows - 1;
#pragma unroll
    for (int c = 0; c < G::DC; c++) {
      if (!PAD || 2 * c + hl < validChunks)
        qf[qi][c] = *reinterpret_cast<const v8 *>(qbase + (size_t)row * tokBytes + (16 * c + 8 * hl) * 2);
      else
        qf[qi][c] = v8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  // ---- operand addresses inside a stage ---------------------------------------
  // K: lane (key l32 [+32kb], d chunk 2c+hl) reads 16 bytes.
  // (k-steps 8 apart read chunks 16 apart: the swizzle leaves that bit alone)
  auto kfragOf = [&](int c, int row32, int half) {
    return (uint32_t)(row32 * G::rowBytes + (((2 * c + half) ^ G::kSwz(row32)) * 16));
  };
  // V: as a source of the transposing read, lane L of a 16-lane group g points
  // at key 4*hl + L/4 (+ 32kb + 16m + 8e), d = 32db + 16*(g%2) + 4*(L%4).
  // (O^T blocks 4 apart read chunks 16 apart)
  auto vfragOf = [&](int db, int ln) {
    const int g = ln / 16, L = ln % 16, r = L % 4, j = L / 4, half = ln / 32;
    const int chunk = (4 * db + 2 * (g % 2) + r / 2) ^ G::vSwz(4 * half + j);
    return (uint32_t)((4 * half + j) * G::rowBytes + chunk * 16 + 8 * (r % 2));
  };
  // (as with the movers' offsets: kept in registers, or recomputed per tile at D = 256)
  uint32_t kfrag[G::KF], vfrag[G::VF];
#pragma unroll
  for (int c = 0; c < G::KF; c++) kfrag[c] = kRecomputeOffsets ? 0u : kfragOf(c, l32, hl);
#pragma unroll
  for (int db = 0; db < G::VF; db++) vfrag[db] = kRecomputeOffsets ? 0u : vfragOf(db, lane);

  f32x16 accO[NQ][G::DB];
  float m_run[NQ], l_run[NQ]; // stale reference maximum (raw score units), this lane's share of the running sum
#pragma unroll
  for (int qi = 0; qi < NQ; qi++) {
    m_run[qi] = 0.0f;
    l_run[qi] = 0.0f;
#pragma unroll
    for (int db = 0; db < G::DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) accO[qi][db][i] = 0.0f;
  }

  // The Q operands arrive through loads the compiler keeps count of.  Where it has not
  // peeled the first tile off the loop, it waits for them at the first score MFMAs inside
  // the loop, with counts that in hardware also cover the direct-to-LDS loads of the next
  // tiles issued just before.  A use of every Q register here puts that wait in front of
  // the loop.  Measured: 2-8 % faster for the causal and the 64-query instances at
  // head_dim 64, no gain at 128 and 256 (two-stage ring: the next tile is mostly in L2).
  constexpr bool kQWaitAhead = D == 64 && (CAUSAL || NQ == 2);
  if (kQWaitAhead) {
#pragma unroll
    for (int qi = 0; qi < NQ; qi++)
#pragma unroll
      for (int c = 0; c < G::DC; c++) asm volatile("" ::"v"(qf[qi][c]));
  }
  for (int kt = 0; kt < nkt; kt++) {
    if (TRACE) tMark = clock64();
    // The loads of tile kt (and of nothing later) must have landed; the barrier
    // makes every wavefront's share visible and also says that everybody is
    // done with tile kt-1, whose stage the next load may overwrite.
    // (with a ring of three, tile kt + 1 may still fly: its 2 * LPW loads)
    if (kStages > 2 && kt + 1 < nkt) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LPW) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (TRACE && kt == 0) tFirstTile = clock64();
    if (kt + kStages - 1 < nkt) issueTile(kt + kStages - 1);

    const uint32_t stageOff = (uint32_t)((kt % kStages) * kStageBytes);
    const int key0 = kt * kBN;

    // Rows of masked keys meet p = 0; zero them so that stray NaN/Inf bits in
    // padding cannot reach the accumulators.  Only the last tile can be partial.
    if (key0 + kBN > kvlen) {
      unsigned char *vst = smem + stageOff + kTileBytes;
#pragma unroll
      for (int i = 0; i < kTileBytes / 4096; i++) {
        const int chunk = tid + 256 * i; // 16-byte chunk of the V tile
        if (key0 + chunk / G::CPR >= kvlen)
          *reinterpret_cast<u32x4 *>(vst + chunk * 16) = u32x4{0u, 0u, 0u, 0u};
      }
      __syncthreads();
    }

    // Causal: a wavefront whose queries all precede this tile has nothing to add.
    if (CAUSAL && key0 > q0 + NQ * 32 - 1) continue;

    // Operand pointers in the LDS address space: one add per tile, the rest
    // of every address is an instruction immediate.
    const lds_u8 *kp[G::KF], *vp[G::VF];
    int ln = lane;
    if (kRecomputeOffsets) asm volatile("" : "+v"(ln));
#pragma unroll
    for (int c = 0; c < G::KF; c++)
      kp[c] = (const lds_u8 *)(uintptr_t)(ldsBase + stageOff + (kRecomputeOffsets ? kfragOf(c, ln % 32, ln / 32) : kfrag[c]));
#pragma unroll
    for (int db = 0; db < G::VF; db++)
      vp[db] = (const lds_u8 *)(uintptr_t)(ldsBase + stageOff + kTileBytes + (kRecomputeOffsets ? vfragOf(db, ln) : vfrag[db]));

    if (TRACE) {
      const uint64_t t = clock64();
      cWait += t - tMark;
      tMark = t;
    }
    // ---- S^T = K Q^T -------------------------------------------------------
    f32x16 accS[NQ][G::KB];
    __builtin_amdgcn_s_setprio(2); // MFMA phases outrank the softmax phases of the SIMD's other wavefronts
#pragma unroll
    for (int kb = 0; kb < G::KB; kb++) {
#pragma unroll
      for (int c = 0; c < G::DC; c++) {
        const v8 a = *reinterpret_cast<const v8 __attribute__((address_space(3))) *>(kp[c % G::KF] + (c / G::KF) * 256 +
                                                                                      kb * 32 * G::rowBytes);
#pragma unroll
        for (int qi = 0; qi < NQ; qi++) {
          if (c == 0) {
#pragma unroll
            for (int i = 0; i < 16; i++) accS[qi][kb][i] = 0.0f;
          }
          accS[qi][kb] = M::run(a, qf[qi][c], accS[qi][kb]);
        }
      }
    }

    __builtin_amdgcn_s_setprio(0);
    if (TRACE) {
      // a use of the last accumulator makes the stamp wait for the MFMAs
      asm volatile("" ::"v"(accS[NQ - 1][G::KB - 1][15]));
      const uint64_t t = clock64();
      cScores += t - tMark;
      tMark = t;
    }
    const bool needMask = (key0 + kBN > kvlen) || (CAUSAL && key0 + kBN - 1 > q0);
    v8 pf[NQ][G::KB][2];
#pragma unroll
    for (int qi = 0; qi < NQ; qi++) {
      if (needMask) {
        const int query = q0 + qi * 32 + l32;
#pragma unroll
        for (int kb = 0; kb < G::KB; kb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int key = key0 + 32 * kb + 8 * (i / 4) + 4 * hl + (i % 4);
            const bool ok = key < kvlen && (!CAUSAL || key <= query);
            if (!ok) accS[qi][kb][i] = -INFINITY;
          }
      }
      // ---- P against the stale reference maximum ---------------------------
      auto makeP = [&](float mref) {
        const float mc = mref * scale_log2e;
        float lsum = 0.0f, lsumOdd = 0.0f;
#pragma unroll
        for (int kb = 0; kb < G::KB; kb++)
#pragma unroll
          for (int m = 0; m < 2; m++) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
              const float e = __builtin_amdgcn_exp2f(accS[qi][kb][8 * m + j] * scale_log2e - mc);
              (j & 1 ? lsumOdd : lsum) += e;
              pf[qi][kb][m][j] = M::narrow(e);
            }
          }
        return lsum + lsumOdd;
      };
      float lsum = makeP(m_run[qi]);
      // Reference too low (P overflows) or too high (everything so far underflows).
      if (__builtin_amdgcn_ballot_w64(!(lsum <= kSumLimit) || (kt == 0 && !(lsum >= kSumFloor))) != 0) {
        float mx = accS[qi][0][0];
#pragma unroll
        for (int kb = 0; kb < G::KB; kb++)
#pragma unroll
          for (int i = 0; i < 16; i++) mx = fmaxf(mx, accS[qi][kb][i]);
        mx = halves_max(mx);
        float m_new, alpha;
        if (kt > 0) { // the row has a history: the reference only rises
          m_new = fmaxf(m_run[qi], mx);
          alpha = __builtin_amdgcn_exp2f((m_run[qi] - m_new) * scale_log2e);
        } else { // first tile: start over from its maximum
          m_new = mx == -INFINITY ? m_run[qi] : mx;
          alpha = 0.0f;
        }
        m_run[qi] = m_new;
        l_run[qi] *= alpha;
#pragma unroll
        for (int db = 0; db < G::DB; db++)
#pragma unroll
          for (int i = 0; i < 16; i++) accO[qi][db][i] *= alpha;
        lsum = makeP(m_new);
      }
      l_run[qi] += lsum;
    }

    if (TRACE) {
      const uint64_t t = clock64();
      cSoftmax += t - tMark;
      tMark = t;
    }
    // ---- O^T += V^T P^T ----------------------------------------------------
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int db = 0; db < G::DB; db++) {
#pragma unroll
      for (int kb = 0; kb < G::KB; kb++) {
#pragma unroll
        for (int m = 0; m < 2; m++) {
          const lds_u8 *p = vp[db % G::VF] + (db / G::VF) * 256 + (32 * kb + 16 * m) * G::rowBytes;
          const v4 lo = M::readTr(p);                    // k-slots 0..3: keys +4hl+0..3
          const v4 hi = M::readTr(p + 8 * G::rowBytes);  // k-slots 4..7: keys +8+4hl+0..3
          const v8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
          for (int qi = 0; qi < NQ; qi++) accO[qi][db] = M::run(a, pf[qi][kb][m], accO[qi][db]);
        }
      }
    }
    __builtin_amdgcn_s_setprio(0);
    if (TRACE) {
      asm volatile("" ::"v"(accO[NQ - 1][G::DB - 1][15]));
      cPV += clock64() - tMark;
    }
  }

  if (TRACE) tLoopEnd = clock64();
  // ---- normalise, transpose through LDS, store whole rows ------------------
  __syncthreads(); // every wavefront is done reading the K / V tiles
  constexpr int kOS = G::OS;
  uint16_t *stage = reinterpret_cast<uint16_t *>(smem) + wave * (NQ * 32 * kOS);
#pragma unroll
  for (int qi = 0; qi < NQ; qi++) {
    const float l = halves_sum(l_run[qi]);
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
    for (int db = 0; db < G::DB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        v4 o;
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = M::narrow(accO[qi][db][4 * g + i] * inv);
        *reinterpret_cast<v4 *>(&stage[(qi * 32 + l32) * kOS + 32 * db + 8 * g + 4 * hl]) = o;
      }
  }
  // Each wavefront reads back only what it wrote: no block barrier needed, the
  // LDS accesses of one wavefront are ordered.
#pragma unroll
  for (int it = 0; it < NQ * 32 * G::CPR / 64; it++) {
    const int chunk = it * 64 + lane; // 16-byte chunk index inside the wave's tile
    const int r = chunk / G::CPR, cidx = chunk % G::CPR;
    const int query = q0 + r;
    if (query < rows && (!PAD || cidx < validChunks)) {
      // 8-byte LDS reads: the staging stride is 8-byte but not 16-byte aligned
      const u32x2 lo = *reinterpret_cast<const u32x2 *>(&stage[r * kOS + cidx * 8]);
      const u32x2 hi = *reinterpret_cast<const u32x2 *>(&stage[r * kOS + cidx * 8 + 4]);
      const u32x4 val = {lo[0], lo[1], hi[0], hi[1]};
      __builtin_nontemporal_store(
          val, reinterpret_cast<u32x4 *>(out + (tok0 + query) * H * kD + (size_t)h * kD + cidx * 8));
    }
  }
  // the next part's tiles land in the ring the staging area sits in
  if (part + 1 < nParts) __syncthreads();
  }; // runPart
  if constexpr (kCanPair) {
#pragma clang loop unroll(disable)
    for (int part = 0; part < nParts; part++) runPart(part);
  } else {
    runPart(0);
  }
  if (TRACE && threadIdx.x == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the output stores have left the wavefront
    uint64_t *rec = stamps + (size_t)blockIdx.x * 10;
    rec[0] = tEntry;
    rec[1] = tFirstTile;
    rec[2] = tLoopEnd;
    rec[3] = clock64();
    rec[4] = wEntry;
    rec[5] = wall_clock64();
    rec[6] = cWait;
    rec[7] = cScores;
    rec[8] = cSoftmax;
    rec[9] = cPV;
  }
}

} // namespace fmha_detail

} // namespace mgpu
