// Fused multi-head attention forward for head_dim 64 on gfx950 MFMA.
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
// queries.  Key/value tiles of BN = 64 keys are staged through LDS (double
// buffered, next tile's global loads in flight while the current one is
// consumed) and shared by the 4 wavefronts.
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
// V is transposed on its way into LDS (4x4 halves in registers, 8-byte writes),
// rows padded so that operand reads are bank-conflict free.
//
// Softmax runs in fp32 in base 2: p = exp2(s*c - m*c), c = scale*log2(e), with
// the usual running maximum / running sum rescaling.
#include "common.hpp"
#include "mgpu_ops_internal.hpp"
#include "types.hpp"

namespace mgpu {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kD = 64;   // head dim
constexpr int kBN = 64;  // keys per tile
constexpr int kKS = 72;  // K tile row stride in elements (144 B: conflict-free 16 B reads)
constexpr int kVS = 68;  // V^T tile row stride in elements (136 B: conflict-free 8 B reads)

template <typename T> struct Mma;
template <> struct Mma<_Float16> {
  using v8 = f16x8;
  using v4 = f16x4;
  __device__ static __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ _Float16 narrow(float f) { return (_Float16)f; }
};
template <> struct Mma<bf16_t> {
  using v8 = bf16x8;
  using v4 = bf16x4;
  __device__ static __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ __bf16 narrow(float f) { return (__bf16)f; }
};

// Exchange with lane l ^ 32: v_permlane32_swap hands every lane the value of
// the lower half in r[0] and of the upper half in r[1].
__device__ __forceinline__ float halves_max(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float halves_sum(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

template <typename T, int NQ, bool CAUSAL>
__global__ __launch_bounds__(256) void fmha_fwd_d64_kernel(const uint16_t *__restrict__ qkv,
                                                           const int32_t *__restrict__ seqlens,
                                                           uint16_t *__restrict__ out, int S, int H,
                                                           int nQB, float scale_log2e) {
  using M = Mma<T>;
  using v8 = typename M::v8;
  using v4 = typename M::v4;
  constexpr int BM = 128 * NQ;

  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][kBN * kKS];
  __shared__ __attribute__((aligned(16))) uint16_t Vt[2][kD * kVS];

  // Work-item order: query blocks of one (batch, head) are consecutive, and a
  // contiguous run of work items goes to each of the 8 XCDs (consecutive block
  // ids are dealt round-robin to the XCDs), so the blocks that re-read the
  // same K/V share one L2.
  const int nblk = gridDim.x;
  const int bid = blockIdx.x;
  const int wid = (nblk % 8 == 0) ? (bid % 8) * (nblk / 8) + bid / 8 : bid;
  const int qb = wid % nQB;
  const int bh = wid / nQB;
  const int h = bh % H;
  const int b = bh / H;

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = tid / 64;
  const int l32 = lane % 32;
  const int hl = lane / 32;

  int kvlen = S;
  if (seqlens) {
    kvlen = seqlens[b];
    kvlen = kvlen < 0 ? 0 : (kvlen > S ? S : kvlen);
  }
  const int q0 = qb * BM + wave * (NQ * 32); // first query of this wavefront
  const size_t tok = (size_t)3 * H * kD;      // elements per token row
  const uint16_t *qbase = qkv + (size_t)b * S * tok + (size_t)h * kD;
  const uint16_t *kbase = qbase + (size_t)H * kD;
  const uint16_t *vbase = qbase + (size_t)2 * H * kD;

  // Q as the B operand: lane (query l32, k-slots = d 16c + 8hl .. +7).
  v8 qf[NQ][4];
#pragma unroll
  for (int qi = 0; qi < NQ; qi++) {
    int row = q0 + qi * 32 + l32;
    row = row < S ? row : S - 1;
#pragma unroll
    for (int c = 0; c < 4; c++)
      qf[qi][c] = *reinterpret_cast<const v8 *>(qbase + (size_t)row * tok + 16 * c + 8 * hl);
  }

  int kend = kvlen;
  if (CAUSAL) {
    int lastq = qb * BM + BM - 1;
    lastq = lastq < S - 1 ? lastq : S - 1;
    kend = kend < lastq + 1 ? kend : lastq + 1;
  }
  const int nkt = (kend + kBN - 1) / kBN;

  // Tile movers.  K: thread -> rows tid/8 and tid/8 + 32, 8 elements at
  // column 8*(tid%8).  V: thread -> rows 4*(tid/16)..+3, 4 elements at column
  // 4*(tid%16), transposed in registers before the LDS write.
  const int krow = tid / 8, kcol = (tid % 8) * 8;
  const int vk0 = 4 * (tid / 16), vd0 = 4 * (tid % 16);
  u32x4 kreg[2];
  u32x2 vreg[4];

  auto loadTile = [&](int kt) {
#pragma unroll
    for (int r = 0; r < 2; r++) {
      int key = kt * kBN + krow + 32 * r;
      key = key < S ? key : S - 1;
      kreg[r] = *reinterpret_cast<const u32x4 *>(kbase + (size_t)key * tok + kcol);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int key = kt * kBN + vk0 + i;
      const int keyc = key < S ? key : S - 1;
      u32x2 v = *reinterpret_cast<const u32x2 *>(vbase + (size_t)keyc * tok + vd0);
      // Rows of masked keys meet p = 0; zero them so that stray NaN/Inf bits in
      // padding cannot reach the accumulators.
      if (key >= kvlen) v = u32x2{0u, 0u};
      vreg[i] = v;
    }
  };
  auto storeTile = [&](int buf) {
#pragma unroll
    for (int r = 0; r < 2; r++)
      *reinterpret_cast<u32x4 *>(&Ks[buf][(krow + 32 * r) * kKS + kcol]) = kreg[r];
    // 4x4 transpose of 16-bit values: word j of the result row for column d
    // packs that column of two consecutive keys.
    constexpr uint32_t LO = 0x05040100u, HI = 0x07060302u;
    u32x2 t[4];
    t[0] = u32x2{__builtin_amdgcn_perm(vreg[1][0], vreg[0][0], LO), __builtin_amdgcn_perm(vreg[3][0], vreg[2][0], LO)};
    t[1] = u32x2{__builtin_amdgcn_perm(vreg[1][0], vreg[0][0], HI), __builtin_amdgcn_perm(vreg[3][0], vreg[2][0], HI)};
    t[2] = u32x2{__builtin_amdgcn_perm(vreg[1][1], vreg[0][1], LO), __builtin_amdgcn_perm(vreg[3][1], vreg[2][1], LO)};
    t[3] = u32x2{__builtin_amdgcn_perm(vreg[1][1], vreg[0][1], HI), __builtin_amdgcn_perm(vreg[3][1], vreg[2][1], HI)};
#pragma unroll
    for (int j = 0; j < 4; j++)
      *reinterpret_cast<u32x2 *>(&Vt[buf][(vd0 + j) * kVS + vk0]) = t[j];
  };

  f32x16 accO[NQ][2];
  float m_run[NQ], l_run[NQ];
#pragma unroll
  for (int qi = 0; qi < NQ; qi++) {
    m_run[qi] = -INFINITY;
    l_run[qi] = 0.0f;
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) accO[qi][db][i] = 0.0f;
  }

  if (nkt > 0) loadTile(0);
  for (int kt = 0; kt < nkt; kt++) {
    const int buf = kt & 1;
    storeTile(buf);
    __syncthreads();
    if (kt + 1 < nkt) loadTile(kt + 1);

    const int key0 = kt * kBN;
    // Causal: a wavefront whose queries all precede this tile has nothing to add.
    if (CAUSAL && key0 > q0 + NQ * 32 - 1) continue;

    // ---- S^T = K Q^T ---------------------------------------------------
    f32x16 accS[NQ][2];
#pragma unroll
    for (int qi = 0; qi < NQ; qi++)
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) accS[qi][kb][i] = 0.0f;
#pragma unroll
    for (int kb = 0; kb < 2; kb++) {
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const v8 a = *reinterpret_cast<const v8 *>(&Ks[buf][(32 * kb + l32) * kKS + 16 * c + 8 * hl]);
#pragma unroll
        for (int qi = 0; qi < NQ; qi++) accS[qi][kb] = M::run(a, qf[qi][c], accS[qi][kb]);
      }
    }

    // ---- online softmax, one query per lane column ------------------------
    const bool needMask = (key0 + kBN > kvlen) || (CAUSAL && key0 + kBN - 1 > q0);
    v8 pf[NQ][2][2];
#pragma unroll
    for (int qi = 0; qi < NQ; qi++) {
      if (needMask) {
        const int query = q0 + qi * 32 + l32;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int key = key0 + 32 * kb + 8 * (i / 4) + 4 * hl + (i % 4);
            const bool ok = key < kvlen && (!CAUSAL || key <= query);
            if (!ok) accS[qi][kb][i] = -INFINITY;
          }
      }
      float mx = accS[qi][0][0];
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) mx = fmaxf(mx, accS[qi][kb][i]);
      mx = halves_max(mx);
      const float m_new = fmaxf(m_run[qi], mx);
      const float alpha = __builtin_amdgcn_exp2f((m_run[qi] - m_new) * scale_log2e);
      const float mc = m_new * scale_log2e;
      float lsum = 0.0f;
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const float p = __builtin_amdgcn_exp2f(accS[qi][kb][i] * scale_log2e - mc);
          accS[qi][kb][i] = p;
          lsum += p;
        }
      l_run[qi] = l_run[qi] * alpha + lsum;
      m_run[qi] = m_new;
#pragma unroll
      for (int db = 0; db < 2; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) accO[qi][db][i] *= alpha;
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int m = 0; m < 2; m++)
#pragma unroll
          for (int j = 0; j < 8; j++) pf[qi][kb][m][j] = M::narrow(accS[qi][kb][8 * m + j]);
    }

    // ---- O^T += V^T P^T ----------------------------------------------------
#pragma unroll
    for (int db = 0; db < 2; db++) {
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int m = 0; m < 2; m++) {
          const uint16_t *vrow = &Vt[buf][(32 * db + l32) * kVS + 32 * kb + 16 * m + 4 * hl];
          const v4 lo = *reinterpret_cast<const v4 *>(vrow);
          const v4 hi = *reinterpret_cast<const v4 *>(vrow + 8);
          const v8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
          for (int qi = 0; qi < NQ; qi++) accO[qi][db] = M::run(a, pf[qi][kb][m], accO[qi][db]);
        }
      }
    }
  }

  // ---- normalise and store -------------------------------------------------
#pragma unroll
  for (int qi = 0; qi < NQ; qi++) {
    const float l = halves_sum(l_run[qi]);
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    const int query = q0 + qi * 32 + l32;
    if (query < S) {
      uint16_t *orow = out + ((size_t)b * S + query) * H * kD + (size_t)h * kD;
#pragma unroll
      for (int db = 0; db < 2; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          v4 o;
#pragma unroll
          for (int i = 0; i < 4; i++) o[i] = M::narrow(accO[qi][db][4 * g + i] * inv);
          *reinterpret_cast<v4 *>(orow + 32 * db + 8 * g + 4 * hl) = o;
        }
    }
  }
}

template <typename T, int NQ>
void launch(const void *qkv, const int32_t *seqlens, void *out, int B, int S, int H, float scale,
            bool causal, hipStream_t stream) {
  constexpr int BM = 128 * NQ;
  const int nQB = (S + BM - 1) / BM;
  const int64_t blocks = (int64_t)B * H * nQB;
  if (blocks > 0x7fffffffLL) fail("fusedMHA: problem too large for one launch");
  const float c = scale * 1.44269504088896340736f;
  const auto *in = static_cast<const uint16_t *>(qkv);
  auto *o = static_cast<uint16_t *>(out);
  if (causal)
    fmha_fwd_d64_kernel<T, NQ, true><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(in, seqlens, o, S, H, nQB, c);
  else
    fmha_fwd_d64_kernel<T, NQ, false><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(in, seqlens, o, S, H, nQB, c);
  MGPU_CHECK_LAUNCH("fmha_fwd_d64_kernel");
}

} // namespace

void fusedMHA(DType dt, const void *qkv, const int32_t *seqlens, void *out, int B, int S, int H,
              int D, float scale, bool causal, hipStream_t stream) {
  if (B < 0 || S < 0 || H < 0) fail("fusedMHA: negative shape");
  if (D != kD) fail("fusedMHA: only head_dim 64 is built");
  if (B == 0 || S == 0 || H == 0) return;
  if (!qkv || !out) fail("fusedMHA: null pointer");
  if (!aligned16(qkv) || !aligned16(out)) fail("fusedMHA: qkv and out must be 16-byte aligned");
  if (!(scale > 0.0f) || !(scale < INFINITY)) fail("fusedMHA: softmax scale must be positive and finite");
  if (dt == DType::F16)
    launch<_Float16, 1>(qkv, seqlens, out, B, S, H, scale, causal, stream);
  else if (dt == DType::BF16)
    launch<bf16_t, 1>(qkv, seqlens, out, B, S, H, scale, causal, stream);
  else
    fail("fusedMHA: element type must be fp16 or bf16");
}

} // namespace mgpu
