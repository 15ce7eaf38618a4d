// A state-space recurrence with a step size and a decay that depend on the token (the "state-space duality" form):
// per sequence and head h, with group g = h / (H / G),
//
//   dt_t = softplus(d_t + dt_bias[h]),   a_t = exp(-exp(A_log[h]) dt_t)
//   S_t  = a_t S_(t-1) + dt_t B_t x_t^T            S is N x P, float32, the request's, zero at its start
//   y_t  = S_t^T C_t + D[h] x_t
//
// x (T, H P), B and C (T, G N each) stand side by side in `xbc` rows (float32: they come from the convolution's
// kernel); d stands in the input product's rows from column `odt` on.  Everything here is float32.
//
//   ssd_scan   token by token: one block per (sequence, head, PC value columns); thread (rg, j) keeps the rows
//              rg, rg + RG, ... of the state's column j in registers; SSD_TS tokens are staged through LDS at a time
//              (B, C, x, dt, a), each thread adds its rows' share of y, and the RG shares of an output are added in
//              ascending order once per staged run.  The sums run in one order whatever the cut: whole prompts,
//              portions and single tokens give the same bits.
#include "common.h"

constexpr int SSD_TS = 8;

__device__ __forceinline__ float ssd_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename TD, int PC, int NK>
__global__ __launch_bounds__(256) void ssd_scan_kernel(const float* __restrict__ xbc, int ldx, int ob, int oc,
                                                       const TD* __restrict__ drows, int ldd, int odt,
                                                       const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                                       const float* __restrict__ d_skip, float* __restrict__ state,
                                                       const int* __restrict__ q_start, const int* __restrict__ slots,
                                                       float* __restrict__ out, int H, int P, int N, int G) {
  constexpr int RG = 256 / PC;
  constexpr int NP = NK * RG;                 // rows of the state a block can hold; B and C are padded to it with zeros
  __shared__ float sB[SSD_TS][NP], sC[SSD_TS][NP], sX[SSD_TS][PC], sDt[SSD_TS], sA[SSD_TS];
  __shared__ float part[SSD_TS][RG][PC];
  const int s = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * PC;
  const int tid = threadIdx.x, j = tid % PC, rg = tid / PC;
  const int g = h / (H / G);
  const int start = q_start[s], len = q_start[s + 1] - start;
  if (len <= 0) return;
  const bool col = j0 + j < P;
  float* st = state + (((size_t)slots[s] * H + h) * N) * P + j0 + j;
  float S[NK];
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int n = rg + k * RG;
    S[k] = (col && n < N) ? st[(size_t)n * P] : 0.f;
  }
  const float rate = expf(a_log[h]), bias = dt_bias[h], skip = d_skip[h];
  for (int t0 = 0; t0 < len; t0 += SSD_TS) {
    const int nt = len - t0 < SSD_TS ? len - t0 : SSD_TS;
    __syncthreads();                          // the run before has been read
    for (int i = tid; i < nt * NP; i += 256) {
      const int ts = i / NP, n = i % NP;
      const float* row = xbc + (size_t)(start + t0 + ts) * ldx;
      sB[ts][n] = n < N ? row[ob + g * N + n] : 0.f;
      sC[ts][n] = n < N ? row[oc + g * N + n] : 0.f;
    }
    for (int i = tid; i < nt * PC; i += 256) {
      const int ts = i / PC, jj = i % PC;
      sX[ts][jj] = j0 + jj < P ? xbc[(size_t)(start + t0 + ts) * ldx + h * P + j0 + jj] : 0.f;
    }
    if (tid < nt) {
      const float dt = ssd_softplus(to_f32(drows[(size_t)(start + t0 + tid) * ldd + odt + h]) + bias);
      sDt[tid] = dt;
      sA[tid] = expf(-rate * dt);
    }
    __syncthreads();
    for (int ts = 0; ts < nt; ++ts) {
      const float a = sA[ts], bx = sDt[ts] * sX[ts][j];
      float y = 0.f;
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        const int n = rg + k * RG;
        S[k] = fmaf(a, S[k], sB[ts][n] * bx);
        y = fmaf(S[k], sC[ts][n], y);
      }
      part[ts][rg][j] = y;
    }
    __syncthreads();
    for (int i = tid; i < nt * PC; i += 256) {
      const int ts = i / PC, jj = i % PC;
      if (j0 + jj >= P) continue;
      float y = 0.f;
#pragma unroll
      for (int r = 0; r < RG; ++r) y += part[ts][r][jj];
      out[(size_t)(start + t0 + ts) * H * P + h * P + j0 + jj] = y + skip * sX[ts][jj];
    }
  }
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int n = rg + k * RG;
    if (col && n < N) st[(size_t)n * P] = S[k];
  }
}

extern "C" int gs_ssd_max_state() { return 512; }

template <typename TD, int PC>
static int ssd_launch(int nk, dim3 grid, hipStream_t stream, const float* xbc, int ldx, int ob, int oc, const TD* drows,
                      int ldd, int odt, const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                      const int* q_start, const int* slots, float* out, int H, int P, int N, int G) {
#define GS_RUN(NK)                                                                                                   \
  ssd_scan_kernel<TD, PC, NK><<<grid, 256, 0, stream>>>(xbc, ldx, ob, oc, drows, ldd, odt, dt_bias, a_log, d_skip, state, \
                                                        q_start, slots, out, H, P, N, G)
  if (nk <= 4) GS_RUN(4);
  else if (nk <= 8) GS_RUN(8);
  else if (nk <= 16) GS_RUN(16);
  else if (nk <= 32) GS_RUN(32);
  else GS_RUN(64);
#undef GS_RUN
  return 0;
}

extern "C" int gs_ssd_scan(const float* xbc, int ldx, int ob, int oc, const void* drows, int d_dtype, int ldd, int odt,
                           const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                           const int* q_start, const int* slots, float* out, int nseq, int H, int P, int N, int G,
                           hipStream_t stream) {
  GS_REQUIRE(nseq >= 0 && H > 0 && P > 0 && N > 0 && G > 0 && H % G == 0, "ssd_scan: bad sizes nseq=%d H=%d P=%d N=%d G=%d", nseq, H, P, N, G);
  GS_REQUIRE(ldx >= H * P && ob >= 0 && oc >= 0 && ob + G * N <= ldx && oc + G * N <= ldx, "ssd_scan: x, B and C do not fit rows of %d", ldx);
  GS_REQUIRE(odt >= 0 && odt + H <= ldd, "ssd_scan: %d step sizes from column %d do not fit rows of %d", H, odt, ldd);
  if (nseq == 0) return 0;
  // narrow heads: 32 columns a block, eight row groups; else 64 columns and four
  const int pc = P <= 32 ? 32 : 64;
  const int rgn = 256 / pc, nk = gs_ceil_div(N, rgn);
  GS_REQUIRE(nk <= 64 && nseq <= 65535 * 32 && H <= 65535, "ssd_scan: a state of %d rows is more than the kernel holds (%d)", N, 64 * rgn);
  dim3 grid(nseq, H, gs_ceil_div(P, pc));
#define GS_GO(TD)                                                                                                     \
  (pc == 32 ? ssd_launch<TD, 32>(nk, grid, stream, xbc, ldx, ob, oc, (const TD*)drows, ldd, odt, dt_bias, a_log, d_skip, \
                                 state, q_start, slots, out, H, P, N, G)                                              \
            : ssd_launch<TD, 64>(nk, grid, stream, xbc, ldx, ob, oc, (const TD*)drows, ldd, odt, dt_bias, a_log, d_skip, \
                                 state, q_start, slots, out, H, P, N, G))
  if (d_dtype == GS_F32)
    GS_GO(float);
  else if (d_dtype == GS_BF16)
    GS_GO(bf16);
  else
    GS_REQUIRE(false, "ssd_scan: unknown dtype %d", d_dtype);
#undef GS_GO
  GS_LAUNCH_CHECK("ssd_scan");
  return 0;
}
