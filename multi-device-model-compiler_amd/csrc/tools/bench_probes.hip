// Ceiling probes for bench.py --ceilings: what this device delivers to the
// simplest possible kernel of each kind, so that the fractions of the nameplate
// peaks reported for the product kernels can be read against what is reachable.
//   * a plain device copy (one 16-byte vector per lane, one block per 256
//     vectors: the geometry of the library's streaming kernels);
//   * the same copy at the grid and byte count of the headline LayerNorm
//     configuration: the cost of launching, filling and draining 1024 blocks;
//   * a loop of register-fed v_mfma_f32_32x32x16_f16 on four independent
//     accumulators, with the shader clock read inside the kernel;
//   * a model of the attention kernel's tile loop at head_dim 64: the real data
//     flow of a 64-key tile (eight score MFMAs fed by ds_read_b128 of a K tile,
//     the softmax of their results - per score one fma, one exp2, one add, half
//     a convert -, eight P.V MFMAs fed by the converted scores and by
//     ds_read_b64_tr_b16 of a V tile), in the product kernel's three phases or
//     as a half-tile software pipeline with every MFMA followed by an eighth of
//     a half softmax, with 32 or 64 queries per wavefront, with and without the
//     product's tile loads (global_load_lds into a ring of three) and block
//     barrier.  No masks, no row-maximum repair, no prologue or epilogue: what
//     the SIMD, the LDS and the clock governor leave of the matrix rate for this
//     mix, in shader clocks per tile and in wall-clock TFLOP/s.
//   * the LDS read rate behind those operand reads: every wavefront of the
//     device re-reads a 16 KiB tile (64 rows of 256 bytes, the head_dim 128
//     geometry and its chunk swizzles) with ds_read_b128 in the K operand
//     pattern, with ds_read_b64_tr_b16 in the V operand pattern, or with plain
//     ds_read_b64.
// Measurement plumbing only: nothing here is part of the kernel library.
#include "bench_timed.hpp"

#include <hip/hip_bf16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void probe_copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst,
                                                          size_t vectors) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < vectors) __builtin_nontemporal_store(src[i], dst + i);
}

// Two streams in, one out: the memory pattern of the elementwise add (the XOR stands in for the add).
__global__ __launch_bounds__(256) void probe_combine_kernel(const u32x4 *__restrict__ a, const u32x4 *__restrict__ b,
                                                             u32x4 *__restrict__ dst, size_t vectors) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < vectors) __builtin_nontemporal_store(a[i] ^ b[i], dst + i);
}

// iters x 4 MFMAs per wavefront; stamps[2 * block] = shader clocks, [2 * block + 1] = constant-rate clocks
// spent by wavefront 0 of the block.
__global__ __launch_bounds__(256) void probe_mfma_kernel(float *__restrict__ sink, uint64_t *__restrict__ stamps,
                                                          int iters) {
  f16x8 a, b;
  for (int i = 0; i < 8; i++) { // values that differ from lane to lane and slot to slot (see probe_fmha_loop_kernel)
    const uint32_t r = (uint32_t)(threadIdx.x * 8 + i) * 2654435761u + blockIdx.x * 40503u;
    a[i] = (_Float16)(((float)(r & 0xffffu) - 32768.0f) * (0.03f / 32768.0f));
    b[i] = (_Float16)(((float)(r >> 16) - 32768.0f) * (0.03f / 32768.0f));
  }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  const uint64_t t0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c3, 0, 0, 0);
  }
  float s = 0.0f;
  for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
  const uint64_t t1 = clock64(), w1 = wall_clock64();
  if (s == 12345.678f) sink[0] = s; // keeps the accumulators alive
  if (threadIdx.x == 0) {
    stamps[2 * blockIdx.x] = t1 - t0;
    stamps[2 * blockIdx.x + 1] = w1 - w0;
  }
}

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef unsigned char __attribute__((address_space(3))) lds_u8;

__device__ __forceinline__ f16x4 probeReadTr(const lds_u8 *p) {
  return __builtin_bit_cast(f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((i16x4 __attribute__((address_space(3))) *)p));
}
__device__ __forceinline__ f32x16 probeMfma(f16x8 a, f16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// The tile loop of the head_dim-64 attention kernel without its bookkeeping.
// PIPE false: per tile 8 score MFMAs, the softmax of the 32 scores of a lane, 8 P.V MFMAs.
// PIPE true:  sixteen groups per tile, each one MFMA per 32-query block, the operand read for
//             the group three groups on and an eighth of the softmax of a 32-key half:
//             [S_b(t), PV_b(t-1)] under softmax(S_a(t)), then [PV_a(t), S_a(t+1)] under
//             softmax(S_b(t)); nothing moves across a group's fence.
// NQ: 32-query blocks per wavefront.  LOADS: each wavefront issues the product's four
// global_load_lds per tile (K and V of a packed [512, 3, 384, 64] tensor, ring of three
// stages) behind s_waitcnt vmcnt(4) and a block barrier.
// stamps[2 * (4 * block + wave)] = shader clocks of the loop, [.. + 1] = constant-rate clocks.
template <bool PIPE, int NQ, bool LOADS>
__global__ __launch_bounds__(256, NQ == 1 ? 3 : 2) void probe_fmha_loop_kernel(float *__restrict__ sink,
                                                                              uint64_t *__restrict__ stamps, int tiles,
                                                                              float c, const char *__restrict__ kv) {
  constexpr int kStageBytes = 16384, kStages = LOADS ? 3 : 2, AHEAD = 3;
  constexpr uint32_t tokBytes = 3 * 384 * 128;
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kStages * kStageBytes];
  // Operand values spread over (-0.25, 0.25), different in every element: a matrix pipeline fed with
  // one repeated constant draws less power and the device then clocks 10-15 % higher than it does on
  // real activations (the product kernel on constant inputs runs 14-17 % faster than on random ones).
  for (int i = threadIdx.x; i < kStages * kStageBytes / 4; i += 256) {
    const uint32_t r = ((uint32_t)i * 2654435761u + blockIdx.x * 40503u) ^ 0x9e3779b9u;
    const _Float16 lo = (_Float16)(((float)(r & 0xffffu) - 32768.0f) * (0.25f / 32768.0f));
    const _Float16 hi = (_Float16)(((float)(r >> 16) - 32768.0f) * (0.25f / 32768.0f));
    reinterpret_cast<uint32_t *>(smem)[i] =
        (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
  }
  __syncthreads();
  const int lane = threadIdx.x % 64, l32 = lane % 32, hl = lane / 32;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const uint32_t ldsBase = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) unsigned char *)smem);
  // operand addresses of the product kernel's head_dim-64 geometry (swizzled chunks)
  uint32_t kfrag[4], vfrag[2];
  for (int cc = 0; cc < 4; cc++) kfrag[cc] = (uint32_t)(l32 * 128 + (((2 * cc + hl) ^ ((l32 >> 1) & 7)) * 16));
  {
    const int g = lane / 16, L = lane % 16, r = L % 4, j = L / 4;
    for (int db = 0; db < 2; db++) {
      const int chunk = (4 * db + 2 * (g % 2) + r / 2) ^ ((((4 * hl + j) >> 1) & 1) << 2);
      vfrag[db] = (uint32_t)((4 * hl + j) * 128 + chunk * 16 + 8 * (r % 2));
    }
  }
  f16x8 qf[NQ][4];
  for (int qi = 0; qi < NQ; qi++)
    for (int cc = 0; cc < 4; cc++)
      for (int i = 0; i < 8; i++) {
        const uint32_t r = (uint32_t)(((lane * 4 + cc) * 8 + i) * 2 + qi) * 2246822519u + threadIdx.x * 97u;
        qf[qi][cc][i] = (_Float16)(((float)(r >> 16) - 32768.0f) * (0.25f / 32768.0f));
      }
  f32x16 accO[NQ][2] = {};
  float l0[NQ] = {}, l1[NQ] = {};
  const float mc = 0.25f * c;
  const f32x16 zero = {};

  auto kOp = [&](uint32_t stage, int half, int cc) -> f16x8 {
    return *reinterpret_cast<const f16x8 __attribute__((address_space(3))) *>(
        (const lds_u8 *)(uintptr_t)(ldsBase + stage + kfrag[cc]) + half * 32 * 128);
  };
  auto vOp = [&](uint32_t stage, int half, int db, int m) -> f16x8 {
    const lds_u8 *p = (const lds_u8 *)(uintptr_t)(ldsBase + stage + 8192 + vfrag[db]) + (32 * half + 16 * m) * 128;
    const f16x4 lo = probeReadTr(p), hi = probeReadTr(p + 8 * 128);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  struct SV { f32x16 v[NQ]; };
  struct PV { f16x8 v[NQ][2]; };
  auto scores = [&](uint32_t stage, int half) {
    SV s;
#pragma unroll
    for (int qi = 0; qi < NQ; qi++) s.v[qi] = zero;
#pragma unroll
    for (int cc = 0; cc < 4; cc++) {
      const f16x8 a = kOp(stage, half, cc);
#pragma unroll
      for (int qi = 0; qi < NQ; qi++) s.v[qi] = probeMfma(a, qf[qi][cc], s.v[qi]);
    }
    return s;
  };
  auto pv = [&](uint32_t stage, int half, const PV &p) {
#pragma unroll
    for (int m = 0; m < 2; m++)
#pragma unroll
      for (int db = 0; db < 2; db++) {
        const f16x8 a = vOp(stage, half, db, m);
#pragma unroll
        for (int qi = 0; qi < NQ; qi++) accO[qi][db] = probeMfma(a, p.v[qi][m], accO[qi][db]);
      }
  };
  // two scores of a 32-key half: fma, exp2, add, convert
  auto chunk = [&](const f32x16 &sc, f16x8(&p)[2], float &a0, float &a1, int j) {
    const float e0 = __builtin_amdgcn_exp2f(sc[2 * j] * c - mc), e1 = __builtin_amdgcn_exp2f(sc[2 * j + 1] * c - mc);
    a0 += e0;
    a1 += e1;
    p[j / 4][(2 * j) % 8] = (_Float16)e0;
    p[j / 4][(2 * j + 1) % 8] = (_Float16)e1;
  };
  auto softmax = [&](const SV &s, PV &p) {
#pragma unroll
    for (int qi = 0; qi < NQ; qi++)
#pragma unroll
      for (int j = 0; j < 8; j++) chunk(s.v[qi], p.v[qi], l0[qi], l1[qi], j);
  };

  // the product kernel's tile movers: 2 K loads + 2 V loads of 1 KiB per wavefront and tile
  const int mrow = lane / 8, mchunk = lane % 8;
  uint32_t koff[2], voff[2];
  for (int i = 0; i < 2; i++) {
    const int row = 8 * (2 * wave + i) + mrow;
    koff[i] = (uint32_t)row * tokBytes + (uint32_t)((mchunk ^ ((row >> 1) & 7)) * 16);
    voff[i] = (uint32_t)row * tokBytes + (uint32_t)((mchunk ^ (((row >> 1) & 1) << 2)) * 16);
  }
  const char *kbase = kv + (size_t)(blockIdx.x % 384) * 128 + 384 * 128; // the K column of one (batch, head)
  const char *vbase = kbase + 384 * 128;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  auto dma16 = [&](uint32_t voffset, const char *sbase, uint32_t ldsAddr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voffset), "s"(sbase), "s"(ldsAddr) : "memory", "m0");
  };
#pragma clang diagnostic pop
  auto issueTile = [&](int kt) { // tiles 0..7 of the 512 tokens, over and over
    const uint32_t kdst = ldsBase + (uint32_t)((kt % 3) * kStageBytes + (2 * wave) * 1024), vdst = kdst + 8192;
    const char *kg = kbase + (size_t)(kt % 8) * 64 * tokBytes, *vg = vbase + (size_t)(kt % 8) * 64 * tokBytes;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      dma16(koff[i], kg, kdst + i * 1024);
      dma16(voff[i], vg, vdst + i * 1024);
    }
  };
  auto stageOf = [&](int t) { return (uint32_t)(LOADS ? t % 3 : t & 1) * kStageBytes; };
  auto arrive = [&](int t) { // tile t has landed for everybody; the stage of tile t - 1 is free for tile t + 2
    if (LOADS) {
      asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      __syncthreads();
      issueTile(t + 2);
    }
  };
  if (LOADS) {
    issueTile(0);
    issueTile(1);
  }
  const uint64_t t0 = clock64(), w0 = wall_clock64();
  if (!PIPE) {
    for (int t = 0; t < tiles; t++) {
      arrive(t);
      const uint32_t stage = stageOf(t);
      SV sa = scores(stage, 0), sb = scores(stage, 1);
      PV pa, pb;
      softmax(sa, pa);
      softmax(sb, pb);
      pv(stage, 0, pa);
      pv(stage, 1, pb);
    }
  } else {
    // Groups 0..7 of tile t: S_b(t) (4), PV_b(t-1) (4), under the softmax of S_a(t); groups 8..15:
    // PV_a(t) (4), S_a(t+1) (4), under the softmax of S_b(t).  Tile t + 1 must have landed before
    // group 12 - AHEAD reads its K operands: the barrier sits at group 8.
    if (LOADS) {
      asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      __syncthreads();
    }
    SV sa = scores(stageOf(0), 0), sb;
    PV pa = {}, pb = {};
#pragma unroll
    for (int qi = 0; qi < NQ; qi++) sb.v[qi] = zero;
    f16x8 aop[16];
    auto loadOp = [&](int g, uint32_t cur, uint32_t prev, uint32_t next) {
      const int i = g % 8;
      if (g < 8) aop[g] = i < 4 ? kOp(cur, 1, i) : vOp(prev, 1, (i - 4) % 2, (i - 4) / 2);
      else aop[g] = i < 4 ? vOp(cur, 0, i % 2, i / 2) : kOp(next, 0, i - 4);
    };
#pragma unroll
    for (int g = 0; g < AHEAD; g++) loadOp(g, stageOf(0), stageOf(0), stageOf(1));
    for (int t = 0; t < tiles; t++) {
      const uint32_t cur = stageOf(t), prev = stageOf(t + kStages - 1), next = stageOf(t + 1), next2 = stageOf(t + 2);
#pragma unroll
      for (int g = 0; g < 16; g++) {
        if (g == 8 && LOADS) { // PV_b(t-1) is done: its stage takes tile t + 2; tile t + 1 has landed
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __syncthreads();
          issueTile(t + 2);
        }
        if (g + AHEAD < 16) loadOp(g + AHEAD, cur, prev, next);
        else loadOp(g + AHEAD - 16, next, cur, next2);
        const int i = g % 8;
#pragma unroll
        for (int qi = 0; qi < NQ; qi++) {
          if (g < 8) {
            if (i < 4) sb.v[qi] = probeMfma(aop[g], qf[qi][i], i == 0 ? zero : sb.v[qi]);
            else accO[qi][(i - 4) % 2] = probeMfma(aop[g], pb.v[qi][(i - 4) / 2], accO[qi][(i - 4) % 2]);
            chunk(sa.v[qi], pa.v[qi], l0[qi], l1[qi], i);
          } else {
            if (i < 4) accO[qi][i % 2] = probeMfma(aop[g], pa.v[qi][i / 2], accO[qi][i % 2]);
            else sa.v[qi] = probeMfma(aop[g], qf[qi][i - 4], i == 4 ? zero : sa.v[qi]);
            chunk(sb.v[qi], pb.v[qi], l0[qi], l1[qi], i);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    accO[0][0][0] += sa.v[0][0] + (float)pb.v[0][0][0] + sa.v[NQ - 1][1] + (float)pb.v[NQ - 1][1][1];
  }
  float s = 0.f;
  for (int qi = 0; qi < NQ; qi++) {
    s += l0[qi] + l1[qi];
    for (int i = 0; i < 16; i++) s += accO[qi][0][i] + accO[qi][1][i];
  }
  if (LOADS) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  const uint64_t t1 = clock64(), w1 = wall_clock64();
  if (s == 12345.678f) sink[0] = s;
  if (lane == 0) {
    stamps[2 * (blockIdx.x * 4 + wave)] = t1 - t0;
    stamps[2 * (blockIdx.x * 4 + wave) + 1] = w1 - w0;
  }
}

// Every wavefront reads a 16 KiB tile `iters` times.  MODE 0: sixteen ds_read_b128, lane = (row
// l % 32 [+32], 16-byte chunk (2c + l / 32) ^ (row & 15)) - the K operand reads of the head_dim 128
// attention tile.  MODE 1: thirty-two ds_read_b64_tr_b16 in that tile's V operand pattern.
// MODE 2: thirty-two ds_read_b64 of consecutive 8-byte pieces.
// stamps[2 * block] = shader clocks, [2 * block + 1] = constant-rate clocks of wavefront 0.
template <int MODE>
__global__ __launch_bounds__(256) void probe_lds_read_kernel(uint32_t *__restrict__ sink, uint64_t *__restrict__ stamps,
                                                              int iters) {
  constexpr int rowBytes = 256;
  __shared__ __attribute__((aligned(1024))) unsigned char tile[16384];
  const int tid = threadIdx.x, lane = tid % 64, l32 = lane % 32, hl = lane / 32;
  for (int i = tid; i < 16384 / 4; i += 256) reinterpret_cast<uint32_t *>(tile)[i] = (uint32_t)i * 2654435761u;
  __syncthreads();
  const uint32_t base = (uint32_t)(uintptr_t)((lds_u8 *)tile);
  uint32_t kf[8], vf[4];
  for (int c = 0; c < 8; c++) kf[c] = base + l32 * rowBytes + (((2 * c + hl) ^ (l32 & 15)) * 16);
  for (int db = 0; db < 4; db++) {
    const int g = lane / 16, L = lane % 16, r = L % 4, row = 4 * hl + L / 4;
    vf[db] = base + row * rowBytes + (((4 * db + 2 * (g % 2) + r / 2) ^ ((row & 3) << 2)) * 16) + 8 * (r % 2);
  }
  // The reads are written as assembly so that nothing but the read itself is issued per
  // operand: the results go nowhere, one s_waitcnt per tile collects them.
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  u32x4 wide = {0u, 0u, 0u, 0u};
  u32x2 narrow = {0u, 0u};
  const uint64_t t0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
    if (MODE == 0) {
#pragma unroll
      for (int c = 0; c < 8; c++) {
        asm volatile("ds_read_b128 %0, %1" : "=v"(wide) : "v"(kf[c]));
        asm volatile("ds_read_b128 %0, %1 offset:8192" : "=v"(wide) : "v"(kf[c]));
      }
    } else if (MODE == 1) {
#pragma unroll
      for (int db = 0; db < 4; db++) { // keys 8 * k8 + 4 * hl + 0..3, k8 = 0..7
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(narrow) : "v"(vf[db]));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:2048" : "=v"(narrow) : "v"(vf[db]));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:4096" : "=v"(narrow) : "v"(vf[db]));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:6144" : "=v"(narrow) : "v"(vf[db]));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:8192" : "=v"(narrow) : "v"(vf[db]));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:10240" : "=v"(narrow) : "v"(vf[db]));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:12288" : "=v"(narrow) : "v"(vf[db]));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:14336" : "=v"(narrow) : "v"(vf[db]));
      }
    } else {
      const uint32_t lin = base + lane * 8;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const uint32_t at = lin + i * 2048;
        asm volatile("ds_read_b64 %0, %1" : "=v"(narrow) : "v"(at));
        asm volatile("ds_read_b64 %0, %1 offset:512" : "=v"(narrow) : "v"(at));
        asm volatile("ds_read_b64 %0, %1 offset:1024" : "=v"(narrow) : "v"(at));
        asm volatile("ds_read_b64 %0, %1 offset:1536" : "=v"(narrow) : "v"(at));
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  const uint64_t t1 = clock64(), w1 = wall_clock64();
  u32x4 acc = {wide[0] ^ narrow[0], wide[1] ^ narrow[1], wide[2], wide[3]};
  if (acc[0] == 0x12345u && acc[1] == 7u) sink[0] = acc[2] ^ acc[3]; // keeps the reads alive
  if (threadIdx.x == 0) {
    stamps[2 * blockIdx.x] = t1 - t0;
    stamps[2 * blockIdx.x + 1] = w1 - w0;
  }
}

using mgpu_bench::timed;

// Element i becomes a hashed value spread evenly over (-amplitude, amplitude).
template <typename T>
__global__ void fill_varied_kernel(T *p, size_t n, float amplitude, uint32_t seed) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    uint32_t r = ((uint32_t)i + seed) * 2654435761u;
    r ^= r >> 15;
    r *= 0x85ebca6bu;
    r ^= r >> 13;
    p[i] = (T)(((float)(r >> 8) - 8388608.0f) * (amplitude / 8388608.0f));
  }
}

} // namespace

extern "C" {

// Fills n elements (dtype 0 fp32, 1 fp16, 2 bf16) with values that differ from element to element,
// spread over (-amplitude, amplitude).  What a timed matrix kernel should be fed: on a repeated
// constant the device draws less power and clocks 10-40 % higher than on real data, by an amount
// that differs from kernel to kernel.  Returns 0, or -1 on a launch error or an unknown dtype.
int mgpuProbeFillVaried(void *p, size_t n, int dtype, float amplitude, unsigned seed, void *stream) {
  hipStream_t s = (hipStream_t)stream;
  const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 4096);
  if (n == 0) return 0;
  if (dtype == 0) fill_varied_kernel<float><<<blocks, 256, 0, s>>>((float *)p, n, amplitude, seed);
  else if (dtype == 1) fill_varied_kernel<_Float16><<<blocks, 256, 0, s>>>((_Float16 *)p, n, amplitude, seed);
  else if (dtype == 2) fill_varied_kernel<__hip_bfloat16><<<blocks, 256, 0, s>>>((__hip_bfloat16 *)p, n, amplitude, seed);
  else return -1;
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// Milliseconds for `steps` copies of `bytes` (a multiple of 16) from src[i % nsets] to dst[i % nsets].
float mgpuProbeCopy(void *const *src, void *const *dst, int nsets, size_t bytes, int steps, int warmup, void *stream) {
  const size_t vectors = bytes / 16;
  const unsigned blocks = (unsigned)((vectors + 255) / 256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return timed(
      [&](unsigned long i) {
        probe_copy_kernel<<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const u32x4 *>(src[i % nsets]),
                                                             static_cast<u32x4 *>(dst[i % nsets]), vectors);
      },
      steps, warmup, s);
}

// Milliseconds for `steps` launches that read `bytes` from a[i % nsets] and from b[i % nsets] and write
// `bytes` to dst[i % nsets].
float mgpuProbeCombine(void *const *a, void *const *b, void *const *dst, int nsets, size_t bytes, int steps, int warmup,
                       void *stream) {
  const size_t vectors = bytes / 16;
  const unsigned blocks = (unsigned)((vectors + 255) / 256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return timed(
      [&](unsigned long i) {
        probe_combine_kernel<<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const u32x4 *>(a[i % nsets]),
                                                                static_cast<const u32x4 *>(b[i % nsets]),
                                                                static_cast<u32x4 *>(dst[i % nsets]), vectors);
      },
      steps, warmup, s);
}

// One launch of `blocks` blocks of four wavefronts, iters x 4 MFMAs each.  Returns the milliseconds
// of the launch; *shaderClocks / *constClocks receive the clocks wavefront 0 of block 0 spent in the
// loop (shader clock and the constant-rate clock); stamps must hold 2 * blocks uint64.
float mgpuProbeMfma(void *sink, void *stamps, int blocks, int iters, uint64_t *shaderClocks, uint64_t *constClocks,
                    void *stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float ms = timed(
      [&](unsigned long) {
        probe_mfma_kernel<<<dim3(blocks), dim3(256), 0, s>>>(static_cast<float *>(sink), static_cast<uint64_t *>(stamps),
                                                            iters);
      },
      1, 1, s);
  uint64_t host[2] = {0, 0};
  if (hipMemcpy(host, stamps, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) return -1.0f;
  *shaderClocks = host[0];
  *constClocks = host[1];
  return ms;
}

// The attention tile-loop model (probe_fmha_loop_kernel) with `blocks` blocks of four wavefronts, `tiles`
// tiles each.  variant: bit 0 = half-tile pipeline instead of phases, bit 1 = 64 instead of 32 queries per
// wavefront, bit 2 = with the tile loads and the block barrier.  kv: a packed [512, 3, 384, 64] fp16 tensor
// (75 497 472 bytes), read only with bit 2.  stamps must hold 8 * blocks uint64.  Returns the milliseconds
// of the launch (< 0 on failure); *shaderClocks / *constClocks receive the mean clocks a wavefront spent in
// the loop.
float mgpuProbeFmhaLoop(void *sink, void *stamps, const void *kv, int blocks, int tiles, int variant,
                        double *shaderClocks, double *constClocks, void *stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto *sk = static_cast<float *>(sink);
  auto *st = static_cast<uint64_t *>(stamps);
  const auto *src = static_cast<const char *>(kv);
  if ((variant & 4) && !src) return -1.0f;
  const dim3 grid(blocks), block(256);
  const float c = 0.18f;
  const float ms = timed(
      [&](unsigned long) {
        switch (variant) {
#define MGPU_PROBE_LOOP(V, PIPE, NQ, LOADS)                                                   \
  case V:                                                                                     \
    probe_fmha_loop_kernel<PIPE, NQ, LOADS><<<grid, block, 0, s>>>(sk, st, tiles, c, src);    \
    break;
          MGPU_PROBE_LOOP(0, false, 1, false)
          MGPU_PROBE_LOOP(1, true, 1, false)
          MGPU_PROBE_LOOP(2, false, 2, false)
          MGPU_PROBE_LOOP(3, true, 2, false)
          MGPU_PROBE_LOOP(4, false, 1, true)
          MGPU_PROBE_LOOP(5, true, 1, true)
          MGPU_PROBE_LOOP(6, false, 2, true)
          MGPU_PROBE_LOOP(7, true, 2, true)
#undef MGPU_PROBE_LOOP
        default:
          break;
        }
      },
      1, 1, s);
  if (ms < 0.0f) return ms;
  const size_t n = (size_t)blocks * 4;
  uint64_t *host = new uint64_t[2 * n];
  float result = ms;
  if (hipMemcpy(host, stamps, sizeof(uint64_t) * 2 * n, hipMemcpyDeviceToHost) == hipSuccess) {
    double a = 0.0, b = 0.0;
    for (size_t i = 0; i < n; i++) {
      a += (double)host[2 * i];
      b += (double)host[2 * i + 1];
    }
    *shaderClocks = a / (double)n;
    *constClocks = b / (double)n;
  } else {
    result = -1.0f;
  }
  delete[] host;
  return result;
}

// Rate of the constant clock behind wall_clock64(), in kHz (0 if the runtime does not say).
// probe_lds_read_kernel: one launch of `blocks` blocks of four wavefronts, each wavefront reading 16 KiB of
// LDS `iters` times.  mode 0 = ds_read_b128 (K operand pattern), 1 = ds_read_b64_tr_b16 (V operand pattern),
// 2 = ds_read_b64.  Returns the milliseconds of the launch (< 0 on failure); *shaderClocks / *constClocks
// receive the clocks wavefront 0 of block 0 spent in its loop; stamps must hold 2 * blocks uint64.
float mgpuProbeLdsRead(void *sink, void *stamps, int blocks, int iters, int mode, uint64_t *shaderClocks,
                       uint64_t *constClocks, void *stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto *sk = static_cast<uint32_t *>(sink);
  auto *st = static_cast<uint64_t *>(stamps);
  if (mode < 0 || mode > 2 || blocks <= 0 || iters <= 0) return -1.0f;
  const float ms = timed(
      [&](unsigned long) {
        if (mode == 0) probe_lds_read_kernel<0><<<dim3(blocks), dim3(256), 0, s>>>(sk, st, iters);
        else if (mode == 1) probe_lds_read_kernel<1><<<dim3(blocks), dim3(256), 0, s>>>(sk, st, iters);
        else probe_lds_read_kernel<2><<<dim3(blocks), dim3(256), 0, s>>>(sk, st, iters);
      },
      1, 1, s);
  uint64_t host[2] = {0, 0};
  if (hipMemcpy(host, stamps, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) return -1.0f;
  *shaderClocks = host[0];
  *constClocks = host[1];
  return ms;
}

int mgpuProbeWallClockKHz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}

} // extern "C"
