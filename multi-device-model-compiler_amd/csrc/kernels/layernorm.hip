// LayerNorm and add-residual + LayerNorm for fp32 / fp16 / bf16 rows.
//
// Replaces generalAddBiasResidualLayerNormOpt2 and its dispatch ladder
// (lib/Kernels/GPU/LayerNorm.cu:138-260,262-466).  The reference keeps the row
// in shared memory, writes the output twice and needs two block barriers; here
// a row lives in the registers of one group of 16/32/64 lanes:
//   one 128-bit coalesced load per vector, statistics in fp32 with a two-pass
//   (mean, then centred sum of squares) reduction over registers and DPP /
//   lane-exchange sums, one 128-bit non-temporal store per vector (plain loads
//   + non-temporal stores measured fastest on MI355X).  One pass over HBM.
// Rows wider than a wavefront can hold live in the registers of a whole block
// (layernorm_block_kernel); rows whose length is not a multiple of the vector
// width, rows beyond 256 x 16 vectors and unaligned pointers take the general
// block-per-row kernel.
#include "common.hpp"
#include "mgpu_ops_internal.hpp"
#include "types.hpp"

namespace mgpu {

namespace {

constexpr int kMaxVPL = 8; // vectors per lane the register kernel is built for

// One group of LANES lanes owns one row: lane l holds vectors l, l+LANES, ...
// (VPL of them, the last ones predicated off when the row is shorter; FULL
// says that the row fills all of them, which removes every predicate and with
// it the branches that would sit between the loads).
template <typename T, int LANES, int VPL, bool RESIDUAL, bool FULL>
__global__ __launch_bounds__(256) void layernorm_rows_kernel(
    const T *__restrict__ input, const T *__restrict__ gamma, const T *__restrict__ beta, T *__restrict__ normed,
    int m, int nArg, int rowStep, float eps, const T *__restrict__ residual, T *__restrict__ sumOut) {
  // Argument order: the first 14 dwords are preloaded into SGPRs, and what the path to the
  // first row load needs comes first; rowStep (rows per trip of the grid) stands in for
  // gridDim, which would be a load from the kernarg segment.  A FULL row has a length the
  // instantiation knows.
  using Tr = ElemTraits<T>;
  constexpr int VEC = Tr::kVec; // elements per 16-byte vector
  constexpr int GROUPS = 256 / LANES;
  const int n = FULL ? LANES * VPL * VEC : nArg;
  const int lane = threadIdx.x % LANES;
  const int group = threadIdx.x / LANES;
  const int nvec = n / VEC;
  const float inv_n = 1.0f / (float)n;

  // gamma and beta do not depend on the row: fetch them once, at the top, so that
  // their latency is not paid between the reductions and the stores (a wavefront
  // usually owns a single row and its run time is one chain of latencies) - but
  // behind the loads of the first row: loads return in order, and the row is what
  // the chain waits for first (fp32 (4096, 768): 4.46 -> 4.27 us).
  const u32x4 *gv = reinterpret_cast<const u32x4 *>(gamma);
  const u32x4 *bv = reinterpret_cast<const u32x4 *>(beta);
  u32x4 graw[VPL], braw[VPL];
  u32x4 raw[VPL], rawr[VPL];
  auto loadRow = [&](int row) {
    const u32x4 *xv = reinterpret_cast<const u32x4 *>(input + (size_t)row * n);
    const u32x4 *rv = RESIDUAL ? reinterpret_cast<const u32x4 *>(residual + (size_t)row * n) : nullptr;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = lane + k * LANES;
      if (FULL || v < nvec) {
        raw[k] = xv[v];
        if (RESIDUAL) rawr[k] = rv[v];
      }
    }
  };
  const int row0 = blockIdx.x * GROUPS + group;
  if (row0 < m) loadRow(row0);
#pragma unroll
  for (int k = 0; k < VPL; k++) {
    const int v = lane + k * LANES;
    if (FULL || v < nvec) {
      graw[k] = gv[v];
      braw[k] = bv[v];
    }
  }

  for (int row = row0; row < m; row += rowStep) {
    if (row != row0) loadRow(row);

    float x[VPL][VEC];
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = lane + k * LANES;
      if (FULL || v < nvec) {
        Tr::unpack(raw[k], x[k]);
        if (RESIDUAL) {
          float r[VEC];
          Tr::unpack(rawr[k], r);
#pragma unroll
          for (int e = 0; e < VEC; e++) x[k][e] += r[e];
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) sum += x[k][e];
      } else {
#pragma unroll
        for (int e = 0; e < VEC; e++) x[k][e] = 0.0f;
      }
    }
    const float mean = group_sum<LANES>(sum) * inv_n;

    float sq = 0.0f;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = lane + k * LANES;
      if (FULL || v < nvec) {
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          const float d = x[k][e] - mean;
          sq += d * d;
        }
      }
    }
    const float var = group_sum<LANES>(sq) * inv_n;
    // v_rsq_f32 (1 ulp) in place of the correctly rounded sqrt and division, two dependent
    // sequences of a dozen instructions in the middle of the wavefront's one chain: fp16
    // (4096, 768) 3.93 -> 3.80 us, (262144, 768) fp32 266 -> 263.5 us, the fp32 headline unchanged.
    const float rstd = __builtin_amdgcn_rsqf(var + eps);

    u32x4 *yv = reinterpret_cast<u32x4 *>(normed + (size_t)row * n);
    u32x4 *sv = (RESIDUAL && sumOut) ? reinterpret_cast<u32x4 *>(sumOut + (size_t)row * n) : nullptr;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = lane + k * LANES;
      if (FULL || v < nvec) {
        float g[VEC], b[VEC], y[VEC];
        Tr::unpack(graw[k], g);
        Tr::unpack(braw[k], b);
        if (RESIDUAL) {
          // The sum is stored rounded to T and the normalised value is taken
          // from that rounded sum, while mean and variance came from the
          // un-rounded fp32 sums (reference dataflow, LayerNorm.cu:203-233).
          // (a caller that has no use for the sum passes no buffer for it)
          const u32x4 packed = Tr::pack(x[k]);
          if (sv) __builtin_nontemporal_store(packed, sv + v);
          Tr::unpack(packed, x[k]);
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) y[e] = (x[k][e] - mean) * rstd * g[e] + b[e];
        __builtin_nontemporal_store(Tr::pack(y), yv + v);
      }
    }
  }
}

// fp32 rows in, 16-bit rows out: the cast of the row (round to nearest even,
// stored to castOut) and its LayerNorm in one pass, with the arithmetic of the
// two-kernel sequence - the statistics and the normalisation are taken from the
// values as rounded to T, in the lane grouping and summation order that
// layernorm_rows_kernel uses for the same width, so the results are the same
// bits.  Lane l of a group holds the 8-element vectors l, l + LANES, ... (two
// 16-byte loads each).
template <typename T, int LANES, int VPL, bool FULL>
__global__ __launch_bounds__(256) void layernorm_cast_rows_kernel(const float *__restrict__ input,
                                                                  const T *__restrict__ gamma,
                                                                  const T *__restrict__ beta, T *__restrict__ castOut,
                                                                  T *__restrict__ normed, int m, int nArg, int rowStep,
                                                                  float eps) {
  using Tr = ElemTraits<T>;
  constexpr int VEC = Tr::kVec; // 8
  constexpr int GROUPS = 256 / LANES;
  const int n = FULL ? LANES * VPL * VEC : nArg; // (arguments: as in layernorm_rows_kernel)
  const int lane = threadIdx.x % LANES;
  const int group = threadIdx.x / LANES;
  const int nvec = n / VEC;
  const float inv_n = 1.0f / (float)n;

  const u32x4 *gv = reinterpret_cast<const u32x4 *>(gamma);
  const u32x4 *bv = reinterpret_cast<const u32x4 *>(beta);
  u32x4 graw[VPL], braw[VPL];
  u32x4 lo[VPL], hi[VPL];
  auto loadRow = [&](int row) {
    const u32x4 *xv = reinterpret_cast<const u32x4 *>(input + (size_t)row * n);
#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = lane + k * LANES;
      if (FULL || v < nvec) {
        lo[k] = xv[2 * v];
        hi[k] = xv[2 * v + 1];
      }
    }
  };
  // (the first row's loads go out ahead of gamma and beta, as in layernorm_rows_kernel)
  const int row0 = blockIdx.x * GROUPS + group;
  if (row0 < m) loadRow(row0);
#pragma unroll
  for (int k = 0; k < VPL; k++) {
    const int v = lane + k * LANES;
    if (FULL || v < nvec) {
      graw[k] = gv[v];
      braw[k] = bv[v];
    }
  }

  for (int row = row0; row < m; row += rowStep) {
    if (row != row0) loadRow(row);

    u32x4 *cv = reinterpret_cast<u32x4 *>(castOut + (size_t)row * n);
    float x[VPL][VEC];
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = lane + k * LANES;
      if (FULL || v < nvec) {
        float a[4], b[4];
        ElemTraits<float>::unpack(lo[k], a);
        ElemTraits<float>::unpack(hi[k], b);
        const float wide[VEC] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
        const u32x4 packed = Tr::pack(wide);
        __builtin_nontemporal_store(packed, cv + v);
        Tr::unpack(packed, x[k]);
#pragma unroll
        for (int e = 0; e < VEC; e++) sum += x[k][e];
      } else {
#pragma unroll
        for (int e = 0; e < VEC; e++) x[k][e] = 0.0f;
      }
    }
    const float mean = group_sum<LANES>(sum) * inv_n;

    float sq = 0.0f;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = lane + k * LANES;
      if (FULL || v < nvec) {
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          const float d = x[k][e] - mean;
          sq += d * d;
        }
      }
    }
    const float var = group_sum<LANES>(sq) * inv_n;
    const float rstd = __builtin_amdgcn_rsqf(var + eps);

    u32x4 *yv = reinterpret_cast<u32x4 *>(normed + (size_t)row * n);
#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = lane + k * LANES;
      if (FULL || v < nvec) {
        float g[VEC], b[VEC], y[VEC];
        Tr::unpack(graw[k], g);
        Tr::unpack(braw[k], b);
#pragma unroll
        for (int e = 0; e < VEC; e++) y[e] = (x[k][e] - mean) * rstd * g[e] + b[e];
        __builtin_nontemporal_store(Tr::pack(y), yv + v);
      }
    }
  }
}

// Rows too wide for one wavefront's registers: the same scheme with a whole
// 256-thread block per row (up to 256 x 16 vectors: 16384 fp32 or 32768
// 16-bit elements), the two reductions finished across the 4 wavefronts
// through LDS.  Still one pass over HBM.  gamma and beta are read where they
// are used (holding them would double the registers of a wide row); with
// ROWS = 2 a block works on two rows at a time, which halves that re-reading
// and the barriers per row and keeps more loads in flight.
template <typename T, int VPL, int ROWS, bool RESIDUAL, bool FULL>
__global__ __launch_bounds__(256) void layernorm_block_kernel(
    const T *__restrict__ input, const T *__restrict__ gamma, const T *__restrict__ beta, T *__restrict__ normed,
    int m, int nArg, int rowStep, float eps, const T *__restrict__ residual, T *__restrict__ sumOut) {
  using Tr = ElemTraits<T>;
  constexpr int VEC = Tr::kVec;
  const int n = FULL ? 256 * VPL * VEC : nArg; // (arguments: as in layernorm_rows_kernel)
  __shared__ float partial[2][ROWS][4];
  const int t = threadIdx.x, wave = t / 64;
  const int nvec = n / VEC;
  const float inv_n = 1.0f / (float)n;
  const u32x4 *gv = reinterpret_cast<const u32x4 *>(gamma);
  const u32x4 *bv = reinterpret_cast<const u32x4 *>(beta);

  for (int row0 = blockIdx.x * ROWS; row0 < m; row0 += rowStep) {
    float x[ROWS][VPL][VEC];
    float sum[ROWS];
    {
      u32x4 raw[ROWS][VPL], rawr[ROWS][VPL];
#pragma unroll
      for (int r = 0; r < ROWS; r++) {
        // a row past the end re-reads the last row; its results are not stored
        const int row = row0 + r < m ? row0 + r : m - 1;
        const u32x4 *xv = reinterpret_cast<const u32x4 *>(input + (size_t)row * n);
        const u32x4 *rv = RESIDUAL ? reinterpret_cast<const u32x4 *>(residual + (size_t)row * n) : nullptr;
#pragma unroll
        for (int k = 0; k < VPL; k++) {
          const int v = t + k * 256;
          if (FULL || v < nvec) {
            raw[r][k] = xv[v];
            if (RESIDUAL) rawr[r][k] = rv[v];
          }
        }
      }
#pragma unroll
      for (int r = 0; r < ROWS; r++) {
        sum[r] = 0.0f;
#pragma unroll
        for (int k = 0; k < VPL; k++) {
          const int v = t + k * 256;
          if (FULL || v < nvec) {
            Tr::unpack(raw[r][k], x[r][k]);
            if (RESIDUAL) {
              float rr[VEC];
              Tr::unpack(rawr[r][k], rr);
#pragma unroll
              for (int e = 0; e < VEC; e++) x[r][k][e] += rr[e];
            }
#pragma unroll
            for (int e = 0; e < VEC; e++) sum[r] += x[r][k][e];
          } else {
#pragma unroll
            for (int e = 0; e < VEC; e++) x[r][k][e] = 0.0f;
          }
        }
      }
    }
    // Two barriers per iteration are enough: a wavefront that writes
    // partial[0] for the next rows has passed the second barrier of this
    // iteration, i.e. every wavefront has read partial[0]; the same holds for
    // partial[1] one barrier on.
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      const float s = group_sum<64>(sum[r]);
      if (t % 64 == 0) partial[0][r][wave] = s;
    }
    __syncthreads();
    float mean[ROWS], sq[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      mean[r] = (partial[0][r][0] + partial[0][r][1] + partial[0][r][2] + partial[0][r][3]) * inv_n;
      sq[r] = 0.0f;
#pragma unroll
      for (int k = 0; k < VPL; k++) {
        const int v = t + k * 256;
        if (FULL || v < nvec) {
#pragma unroll
          for (int e = 0; e < VEC; e++) {
            const float d = x[r][k][e] - mean[r];
            sq[r] += d * d;
          }
        }
      }
      const float s = group_sum<64>(sq[r]);
      if (t % 64 == 0) partial[1][r][wave] = s;
    }
    __syncthreads();
    float rstd[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      const float var = (partial[1][r][0] + partial[1][r][1] + partial[1][r][2] + partial[1][r][3]) * inv_n;
      rstd[r] = __builtin_amdgcn_rsqf(var + eps);
    }

#pragma unroll
    for (int k = 0; k < VPL; k++) {
      const int v = t + k * 256;
      if (FULL || v < nvec) {
        float g[VEC], b[VEC];
        Tr::unpack(gv[v], g);
        Tr::unpack(bv[v], b);
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
          if (row0 + r >= m) continue;
          u32x4 *yv = reinterpret_cast<u32x4 *>(normed + (size_t)(row0 + r) * n);
          float y[VEC];
          if (RESIDUAL) { // rounded sum out, normalised value from the rounded sum (see above)
            const u32x4 packed = Tr::pack(x[r][k]);
            if (sumOut) __builtin_nontemporal_store(packed, reinterpret_cast<u32x4 *>(sumOut + (size_t)(row0 + r) * n) + v);
            Tr::unpack(packed, x[r][k]);
          }
#pragma unroll
          for (int e = 0; e < VEC; e++) y[e] = (x[r][k][e] - mean[r]) * rstd[r] * g[e] + b[e];
          __builtin_nontemporal_store(Tr::pack(y), yv + v);
        }
      }
    }
  }
}

// Any n, any alignment: one 256-thread block per row, three sweeps over the
// row (the second and third hit in cache).
template <typename T, bool RESIDUAL>
__global__ __launch_bounds__(256) void layernorm_general_kernel(
    const T *__restrict__ input, const T *__restrict__ gamma, const T *__restrict__ beta, T *__restrict__ normed,
    int m, int n, int rowStep, float eps, const T *__restrict__ residual, T *__restrict__ sumOut) {
  using Tr = ElemTraits<T>;
  __shared__ float partial[4];
  const int wave = threadIdx.x / 64;
  const float inv_n = 1.0f / (float)n;
  for (int row = blockIdx.x; row < m; row += rowStep) {
    const T *xr = input + (size_t)row * n;
    const T *rr = RESIDUAL ? residual + (size_t)row * n : nullptr;
    auto value = [&](int i) {
      float v = Tr::toFloat(xr[i]);
      if (RESIDUAL) v += Tr::toFloat(rr[i]);
      return v;
    };
    float sum = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) sum += value(i);
    sum = group_sum<64>(sum);
    __syncthreads();
    if (threadIdx.x % 64 == 0) partial[wave] = sum;
    __syncthreads();
    const float mean = (partial[0] + partial[1] + partial[2] + partial[3]) * inv_n;
    float sq = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) {
      const float d = value(i) - mean;
      sq += d * d;
    }
    sq = group_sum<64>(sq);
    __syncthreads();
    if (threadIdx.x % 64 == 0) partial[wave] = sq;
    __syncthreads();
    const float var = (partial[0] + partial[1] + partial[2] + partial[3]) * inv_n;
    const float rstd = __builtin_amdgcn_rsqf(var + eps);
    for (int i = threadIdx.x; i < n; i += 256) {
      float v = value(i);
      if (RESIDUAL) {
        const T rounded = Tr::fromFloat(v);
        if (sumOut) sumOut[(size_t)row * n + i] = rounded;
        v = Tr::toFloat(rounded);
      }
      normed[(size_t)row * n + i] =
          Tr::fromFloat((v - mean) * rstd * Tr::toFloat(gamma[i]) + Tr::toFloat(beta[i]));
    }
  }
}

template <typename T, int LANES, int VPL, bool RESIDUAL>
void launchRows(const T *input, const T *residual, const T *gamma, const T *beta, T *sumOut,
                T *normed, float eps, int m, int n, hipStream_t stream) {
  constexpr int GROUPS = 256 / LANES;
  int64_t blocks = ((int64_t)m + GROUPS - 1) / GROUPS;
  const int64_t cap = kMaxStreamBlocks;
  if (blocks > cap) blocks = cap;
  if (n / ElemTraits<T>::kVec == LANES * VPL)
    layernorm_rows_kernel<T, LANES, VPL, RESIDUAL, true><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        input, gamma, beta, normed, m, n, (int)(blocks * GROUPS), eps, residual, sumOut);
  else
    layernorm_rows_kernel<T, LANES, VPL, RESIDUAL, false><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
        input, gamma, beta, normed, m, n, (int)(blocks * GROUPS), eps, residual, sumOut);
  MGPU_CHECK_LAUNCH("layernorm_rows_kernel");
}

template <typename T, int LANES, bool RESIDUAL>
void dispatchVPL(int vpl, const T *input, const T *residual, const T *gamma, const T *beta,
                 T *sumOut, T *normed, float eps, int m, int n, hipStream_t stream) {
  switch (vpl) {
#define MGPU_LN_CASE(V)                                                                          \
  case V:                                                                                        \
    launchRows<T, LANES, V, RESIDUAL>(input, residual, gamma, beta, sumOut, normed, eps, m, n,   \
                                      stream);                                                   \
    break;
    MGPU_LN_CASE(1)
    MGPU_LN_CASE(2)
    MGPU_LN_CASE(3)
    MGPU_LN_CASE(4)
    MGPU_LN_CASE(5)
    MGPU_LN_CASE(6)
    MGPU_LN_CASE(7)
    MGPU_LN_CASE(8)
#undef MGPU_LN_CASE
  default:
    fail("layerNorm: internal dispatch error");
  }
}

template <typename T, bool RESIDUAL>
void layerNormTyped(const T *input, const T *residual, const T *gamma, const T *beta, T *sumOut,
                    T *normed, float eps, int m, int n, hipStream_t stream) {
  constexpr int VEC = ElemTraits<T>::kVec;
  const bool vectorOk = n % VEC == 0 && aligned16(input) && aligned16(gamma) && aligned16(beta) &&
                        aligned16(normed) && (!RESIDUAL || (aligned16(residual) && aligned16(sumOut)));
  const int nvec = n / VEC;
  if (vectorOk && nvec <= 64 * kMaxVPL) {
    // Smallest lane group that keeps at most 4 vectors per lane; wider rows
    // use the whole wavefront with up to kMaxVPL vectors per lane.
    if (nvec <= 16 * 4)
      dispatchVPL<T, 16, RESIDUAL>((nvec + 15) / 16, input, residual, gamma, beta, sumOut, normed,
                                   eps, m, n, stream);
    else if (nvec <= 32 * 4)
      dispatchVPL<T, 32, RESIDUAL>((nvec + 31) / 32, input, residual, gamma, beta, sumOut, normed,
                                   eps, m, n, stream);
    else
      dispatchVPL<T, 64, RESIDUAL>((nvec + 63) / 64, input, residual, gamma, beta, sumOut, normed,
                                   eps, m, n, stream);
    return;
  }
  int64_t blocks = m;
  const int64_t cap = kMaxStreamBlocks;
  if (blocks > cap) blocks = cap;
  if (vectorOk && nvec <= 256 * 16) {
    // smallest of 4 / 8 / 12 / 16 vectors per thread that holds the row; two
    // rows per block at a time while they fit the registers of three or four
    // blocks per CU (fp32 up to 8 vectors, 16-bit types up to 4)
    const int vpl = nvec <= 256 * 4 ? 4 : nvec <= 256 * 8 ? 8 : nvec <= 256 * 12 ? 12 : 16;
    const bool full = nvec == 256 * vpl;
    const bool pairRows = m >= 2 && vpl * ElemTraits<T>::kVec <= 32;
    if (pairRows) blocks = (blocks + 1) / 2;
#define MGPU_LN_BLOCK(V, R, F)                                                                    \
  layernorm_block_kernel<T, V, R, RESIDUAL, F><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>( \
      input, gamma, beta, normed, m, n, (int)(blocks * R), eps, residual, sumOut)
    if (vpl == 4 && pairRows) {
      if (full) MGPU_LN_BLOCK(4, 2, true); else MGPU_LN_BLOCK(4, 2, false);
    } else if (vpl == 4) {
      if (full) MGPU_LN_BLOCK(4, 1, true); else MGPU_LN_BLOCK(4, 1, false);
    } else if (vpl == 8 && pairRows) {
      if (full) MGPU_LN_BLOCK(8, 2, true); else MGPU_LN_BLOCK(8, 2, false);
    } else if (vpl == 8) {
      if (full) MGPU_LN_BLOCK(8, 1, true); else MGPU_LN_BLOCK(8, 1, false);
    } else if (vpl == 12) {
      if (full) MGPU_LN_BLOCK(12, 1, true); else MGPU_LN_BLOCK(12, 1, false);
    } else {
      if (full) MGPU_LN_BLOCK(16, 1, true); else MGPU_LN_BLOCK(16, 1, false);
    }
#undef MGPU_LN_BLOCK
    MGPU_CHECK_LAUNCH("layernorm_block_kernel");
    return;
  }
  layernorm_general_kernel<T, RESIDUAL><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
      input, gamma, beta, normed, m, n, (int)blocks, eps, residual, sumOut);
  MGPU_CHECK_LAUNCH("layernorm_general_kernel");
}

template <typename T>
void layerNormDispatch(const void *input, const void *residual, const void *gamma,
                       const void *beta, void *sumOut, void *normed, float eps, int m, int n,
                       hipStream_t stream) {
  if (residual)
    layerNormTyped<T, true>(static_cast<const T *>(input), static_cast<const T *>(residual),
                            static_cast<const T *>(gamma), static_cast<const T *>(beta),
                            static_cast<T *>(sumOut), static_cast<T *>(normed), eps, m, n, stream);
  else
    layerNormTyped<T, false>(static_cast<const T *>(input), nullptr, static_cast<const T *>(gamma),
                             static_cast<const T *>(beta), nullptr, static_cast<T *>(normed), eps,
                             m, n, stream);
}

} // namespace

void layerNorm(DType dt, const void *input, const void *residual, const void *gamma,
               const void *beta, void *sumOut, void *normed, float eps, int m, int n,
               hipStream_t stream) {
  if (m < 0 || n < 0) fail("layerNorm: negative shape");
  if (m == 0 || n == 0) return;
  if (!input || !gamma || !beta || !normed) fail("layerNorm: null pointer");
  if (sumOut && !residual) fail("layerNorm: a sum output needs a residual");
  switch (dt) {
  case DType::F32:
    layerNormDispatch<float>(input, residual, gamma, beta, sumOut, normed, eps, m, n, stream);
    break;
  case DType::F16:
    layerNormDispatch<_Float16>(input, residual, gamma, beta, sumOut, normed, eps, m, n, stream);
    break;
  case DType::BF16:
    layerNormDispatch<bf16_t>(input, residual, gamma, beta, sumOut, normed, eps, m, n, stream);
    break;
  }
}

bool castLayerNormF32ToF16(const float *input, const void *gamma, const void *beta, void *castOut, void *normed,
                           float eps, int m, int n, hipStream_t stream) {
  if (m < 0 || n < 0) fail("castLayerNorm: negative shape");
  if (m == 0 || n == 0) return true;
  if (!input || !gamma || !beta || !castOut || !normed) fail("castLayerNorm: null pointer");
  const int nvec = n / 8;
  if (n % 8 || nvec > 64 * kMaxVPL || !aligned16(input) || !aligned16(gamma) || !aligned16(beta) ||
      !aligned16(castOut) || !aligned16(normed))
    return false;
  // lane group and vectors per lane as layerNormTyped picks them for fp16 rows
  const int lanes = nvec <= 16 * 4 ? 16 : nvec <= 32 * 4 ? 32 : 64;
  const int vpl = (nvec + lanes - 1) / lanes;
  const bool full = nvec == lanes * vpl;
  int64_t blocks = ((int64_t)m * lanes + 255) / 256;
  if (blocks > kMaxStreamBlocks) blocks = kMaxStreamBlocks;
  const auto *g = static_cast<const _Float16 *>(gamma);
  const auto *b = static_cast<const _Float16 *>(beta);
  auto *c = static_cast<_Float16 *>(castOut);
  auto *y = static_cast<_Float16 *>(normed);
#define MGPU_LN_CAST(L, V)                                                                                     \
  if (lanes == L && vpl == V) {                                                                                \
    if (full)                                                                                                  \
      layernorm_cast_rows_kernel<_Float16, L, V, true><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(      \
          input, g, b, c, y, m, n, (int)(blocks * (256 / L)), eps);                                            \
    else                                                                                                       \
      layernorm_cast_rows_kernel<_Float16, L, V, false><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(     \
          input, g, b, c, y, m, n, (int)(blocks * (256 / L)), eps);                                            \
  }
  MGPU_LN_CAST(16, 1) MGPU_LN_CAST(16, 2) MGPU_LN_CAST(16, 3) MGPU_LN_CAST(16, 4)
  MGPU_LN_CAST(32, 3) MGPU_LN_CAST(32, 4)
  MGPU_LN_CAST(64, 3) MGPU_LN_CAST(64, 4) MGPU_LN_CAST(64, 5) MGPU_LN_CAST(64, 6) MGPU_LN_CAST(64, 7) MGPU_LN_CAST(64, 8)
#undef MGPU_LN_CAST
  MGPU_CHECK_LAUNCH("layernorm_cast_rows_kernel");
  return true;
}

} // namespace mgpu
