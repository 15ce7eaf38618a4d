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
//   ssd_scan   token by token: one block per (sequence, head, PC value columns); thread (rg, j) keeps NK consecutive
//              rows of the state's column j in registers; SSD_TS tokens are staged through LDS at a time (B, C, x, dt,
//              a), each thread adds its rows' share of y, and the RG shares of an output are added in ascending order
//              once per staged run.  The sums run in one order whatever the cut: whole prompts, portions and single
//              tokens give the same bits.
//
// A step that brings long portions leaves most of the chip idle that way (one block a sequence and head walks thousands
// of tokens).  Then the portions are cut into segments (a table made on the host: sequence, first token within the
// portion, tokens, whether it is the portion's last) and three launches do the work:
//   (1) MODE 1: every segment but a portion's last, by a block of its own, from an empty state, without outputs: what
//       the segment's tokens add to the state, G[p], and the product of its decays, A[p], go to a workspace;
//   (2) ssd_combine walks a sequence's segments in order, S[p + 1] = A[p] S[p] + G[p] from the request's own state,
//       and leaves every segment's first state in the workspace (in G's place);
//   (3) MODE 2: every segment from its first state, with outputs; a portion's last segment leaves the request's state.
// The same arithmetic in another association: results differ from the walk in one piece by float32 rounding.
#include "common.h"

constexpr int SSD_TS = 8;

__device__ __forceinline__ float ssd_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename TD, int PC, int NK, int MODE>
__global__ __launch_bounds__(256) void ssd_scan_kernel(const float* __restrict__ xbc, int ldx, int ob, int oc,
                                                       const TD* __restrict__ drows, int ldd, int odt,
                                                       const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                                       const float* __restrict__ d_skip, float* __restrict__ state,
                                                       const int* __restrict__ q_start, const int* __restrict__ slots,
                                                       float* __restrict__ out, int H, int P, int N, int G,
                                                       const int* __restrict__ segs, float* __restrict__ ws,
                                                       float* __restrict__ ws_decay) {
  constexpr int RG = 256 / PC;
  constexpr int NP = NK * RG;                 // rows of the state a block can hold; B and C are padded to it with zeros
  __shared__ __align__(16) float sB[SSD_TS][NP];
  __shared__ __align__(16) float sC[SSD_TS][NP];
  __shared__ float sX[SSD_TS][PC], sDt[SSD_TS], sA[SSD_TS];
  __shared__ float part[SSD_TS][RG][PC];
  const int h = blockIdx.y, j0 = blockIdx.z * PC;
  const int tid = threadIdx.x, j = tid % PC, rg = tid / PC;
  const int g = h / (H / G);
  int s, start, len, last = 1;
  if (MODE == 0) {
    s = blockIdx.x;
    start = q_start[s];
    len = q_start[s + 1] - start;
  } else {
    const int* e = segs + 4 * blockIdx.x;
    s = e[0];
    start = q_start[s] + e[1];
    len = e[2];
    last = e[3];
    if (MODE == 1 && last) return;            // nobody needs what a portion's last segment adds, apart from (3)
  }
  if (len <= 0) return;
  const bool col = j0 + j < P;
  // MODE 0: the request's state, read and left in its slot.  MODE 1: from nothing, left in the workspace.  MODE 2: from
  // the workspace; a portion's last segment leaves the request's state
  float* slot_st = state + (((size_t)slots[s] * H + h) * N) * P + j0 + j;
  float* ws_st = MODE == 0 ? nullptr : ws + (((size_t)blockIdx.x * H + h) * N) * P + j0 + j;
  float S[NK];
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int n = rg * NK + k;
    S[k] = (MODE != 1 && col && n < N) ? (MODE == 0 ? slot_st : ws_st)[(size_t)n * P] : 0.f;
  }
  const float rate = expf(a_log[h]), bias = dt_bias[h], skip = d_skip[h];
  float all_a = 1.f;
  for (int t0 = 0; t0 < len; t0 += SSD_TS) {
    const int nt = len - t0 < SSD_TS ? len - t0 : SSD_TS;
    __syncthreads();                          // the run before has been read
    for (int i = tid; i < nt * NP; i += 256) {
      const int ts = i / NP, n = i % NP;
      const float* row = xbc + (size_t)(start + t0 + ts) * ldx;
      sB[ts][n] = n < N ? row[ob + g * N + n] : 0.f;
      if (MODE != 1) sC[ts][n] = n < N ? row[oc + g * N + n] : 0.f;
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
      const float4* b4 = reinterpret_cast<const float4*>(&sB[ts][rg * NK]);
      const float4* c4 = reinterpret_cast<const float4*>(&sC[ts][rg * NK]);
      float y0 = 0.f, y1 = 0.f;
#pragma unroll
      for (int k = 0; k < NK; k += 4) {
        const float4 b = b4[k / 4];
        S[k] = fmaf(a, S[k], b.x * bx);
        S[k + 1] = fmaf(a, S[k + 1], b.y * bx);
        S[k + 2] = fmaf(a, S[k + 2], b.z * bx);
        S[k + 3] = fmaf(a, S[k + 3], b.w * bx);
        if (MODE != 1) {
          const float4 c = c4[k / 4];
          y0 = fmaf(S[k], c.x, y0);
          y1 = fmaf(S[k + 1], c.y, y1);
          y0 = fmaf(S[k + 2], c.z, y0);
          y1 = fmaf(S[k + 3], c.w, y1);
        }
      }
      if (MODE != 1) part[ts][rg][j] = y0 + y1;
      if (MODE == 1) all_a *= a;
    }
    if (MODE != 1) {
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
  }
  if (MODE == 2 && !last) return;
  float* dst = MODE == 1 ? ws_st : slot_st;
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int n = rg * NK + k;
    if (col && n < N) dst[(size_t)n * P] = S[k];
  }
  if (MODE == 1 && tid == 0 && blockIdx.z == 0) ws_decay[(size_t)blockIdx.x * H + h] = all_a;
}

// One thread per element of a (sequence, head)'s state: the first state of every segment, in order.
__global__ void ssd_combine_kernel(const float* __restrict__ state, const int* __restrict__ slots,
                                   const int* __restrict__ seg_first, float* __restrict__ ws,
                                   const float* __restrict__ ws_decay, int H, int NPn) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * blockDim.x + threadIdx.x;
  if (e >= NPn) return;
  float S = state[((size_t)slots[s] * H + h) * NPn + e];
  const int p1 = seg_first[s + 1];
  for (int p = seg_first[s]; p < p1; ++p) {
    float* w = ws + ((size_t)p * H + h) * NPn + e;
    if (p + 1 < p1) {
      const float add = *w;
      *w = S;
      S = fmaf(ws_decay[(size_t)p * H + h], S, add);
    } else {
      *w = S;
    }
  }
}

// The most state rows a head of P value columns may have: 64 a thread, eight row groups for narrow heads, else four.
extern "C" int gs_ssd_max_state(int P) { return 64 * (P <= 32 ? 8 : 4); }

template <typename TD, int PC, int MODE>
static int ssd_launch(int nk, dim3 grid, hipStream_t stream, const float* xbc, int ldx, int ob, int oc, const TD* drows,
                      int ldd, int odt, const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                      const int* q_start, const int* slots, float* out, int H, int P, int N, int G, const int* segs,
                      float* ws, float* ws_decay) {
#define GS_RUN(NK)                                                                                                    \
  ssd_scan_kernel<TD, PC, NK, MODE><<<grid, 256, 0, stream>>>(xbc, ldx, ob, oc, drows, ldd, odt, dt_bias, a_log, d_skip, \
                                                              state, q_start, slots, out, H, P, N, G, segs, ws, ws_decay)
  if (nk <= 4) GS_RUN(4);
  else if (nk <= 8) GS_RUN(8);
  else if (nk <= 16) GS_RUN(16);
  else if (nk <= 32) GS_RUN(32);
  else GS_RUN(64);
#undef GS_RUN
  return 0;
}

template <int MODE>
static int ssd_go(int d_dtype, int pc, int nk, dim3 grid, hipStream_t stream, const float* xbc, int ldx, int ob, int oc,
                  const void* drows, int ldd, int odt, const float* dt_bias, const float* a_log, const float* d_skip,
                  float* state, const int* q_start, const int* slots, float* out, int H, int P, int N, int G,
                  const int* segs, float* ws, float* ws_decay) {
#define GS_GO(TD, PC)                                                                                                 \
  ssd_launch<TD, PC, MODE>(nk, grid, stream, xbc, ldx, ob, oc, (const TD*)drows, ldd, odt, dt_bias, a_log, d_skip, state, \
                           q_start, slots, out, H, P, N, G, segs, ws, ws_decay)
  if (d_dtype == GS_F32) return pc == 32 ? GS_GO(float, 32) : GS_GO(float, 64);
  if (d_dtype == GS_BF16) return pc == 32 ? GS_GO(bf16, 32) : GS_GO(bf16, 64);
#undef GS_GO
  GS_REQUIRE(false, "ssd_scan: unknown dtype %d", d_dtype);
  return 0;
}

static int ssd_check(int nseq, int H, int P, int N, int G, int ldx, int ob, int oc, int ldd, int odt, int* pc, int* nk) {
  GS_REQUIRE(nseq >= 0 && H > 0 && P > 0 && N > 0 && G > 0 && H % G == 0, "ssd_scan: bad sizes nseq=%d H=%d P=%d N=%d G=%d", nseq, H, P, N, G);
  GS_REQUIRE(ldx >= H * P && ob >= 0 && oc >= 0 && ob + G * N <= ldx && oc + G * N <= ldx, "ssd_scan: x, B and C do not fit rows of %d", ldx);
  GS_REQUIRE(odt >= 0 && odt + H <= ldd, "ssd_scan: %d step sizes from column %d do not fit rows of %d", H, odt, ldd);
  // narrow heads: 32 columns a block, eight row groups; else 64 columns and four
  *pc = P <= 32 ? 32 : 64;
  const int rgn = 256 / *pc;
  *nk = gs_ceil_div(N, rgn);
  GS_REQUIRE(*nk <= 64 && nseq <= 65535 * 32 && H <= 65535, "ssd_scan: a state of %d rows is more than the kernel holds (%d)", N, 64 * rgn);
  return 0;
}

extern "C" int gs_ssd_scan(const float* xbc, int ldx, int ob, int oc, const void* drows, int d_dtype, int ldd, int odt,
                           const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                           const int* q_start, const int* slots, float* out, int nseq, int H, int P, int N, int G,
                           hipStream_t stream) {
  int pc, nk;
  if (int rc = ssd_check(nseq, H, P, N, G, ldx, ob, oc, ldd, odt, &pc, &nk)) return rc;
  if (nseq == 0) return 0;
  dim3 grid(nseq, H, gs_ceil_div(P, pc));
  if (int rc = ssd_go<0>(d_dtype, pc, nk, grid, stream, xbc, ldx, ob, oc, drows, ldd, odt, dt_bias, a_log, d_skip, state,
                         q_start, slots, out, H, P, N, G, nullptr, nullptr, nullptr))
    return rc;
  GS_LAUNCH_CHECK("ssd_scan");
  return 0;
}

// The same over portions cut into segments: `seg_first` (nseq + 1) says where each sequence's segments begin in `segs`
// (nsegs x 4: sequence, first token within the portion, tokens, 1 at a portion's last segment); `ws` holds nsegs x H x
// N x P floats, `ws_decay` nsegs x H.
extern "C" int gs_ssd_scan_segments(const float* xbc, int ldx, int ob, int oc, const void* drows, int d_dtype, int ldd,
                                    int odt, const float* dt_bias, const float* a_log, const float* d_skip, float* state,
                                    const int* q_start, const int* slots, float* out, int nseq, int H, int P, int N, int G,
                                    const int* seg_first, const int* segs, int nsegs, float* ws, float* ws_decay,
                                    hipStream_t stream) {
  int pc, nk;
  if (int rc = ssd_check(nseq, H, P, N, G, ldx, ob, oc, ldd, odt, &pc, &nk)) return rc;
  GS_REQUIRE(nsegs >= nseq && nsegs <= 65535 * 32768, "ssd_scan_segments: %d segments for %d sequences", nsegs, nseq);
  if (nseq == 0) return 0;
  dim3 grid(nsegs, H, gs_ceil_div(P, pc));
  if (nsegs > nseq) {
    if (int rc = ssd_go<1>(d_dtype, pc, nk, grid, stream, xbc, ldx, ob, oc, drows, ldd, odt, dt_bias, a_log, d_skip, state,
                           q_start, slots, out, H, P, N, G, segs, ws, ws_decay))
      return rc;
    GS_LAUNCH_CHECK("ssd_scan_segments (1)");
  }
  ssd_combine_kernel<<<dim3(nseq, H, gs_ceil_div(N * P, 256)), 256, 0, stream>>>(state, slots, seg_first, ws, ws_decay, H, N * P);
  GS_LAUNCH_CHECK("ssd_combine");
  if (int rc = ssd_go<2>(d_dtype, pc, nk, grid, stream, xbc, ldx, ob, oc, drows, ldd, odt, dt_bias, a_log, d_skip, state,
                         q_start, slots, out, H, P, N, G, segs, ws, ws_decay))
    return rc;
  GS_LAUNCH_CHECK("ssd_scan_segments (3)");
  return 0;
}
