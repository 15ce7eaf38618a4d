// Recurrences through a matrix state whose decay depends on the token, with or without the delta rule.
//
// Per sequence and head a state S (n x m, float32, in the request's slot) is advanced token by token:
//
//   S <- diag(a_t) S                      a_t: one number per (token, head), or one per (token, head, key channel)
//   u_t = beta_t (v_t - S^T k_t)          with `delta` (the delta rule: what the state already answers to k_t is taken
//                                         off the value before it is written);  u_t = v_t without
//   S <- S + k_t u_t^T,   o_t = S^T (q_scale q_t)
//
// q_t, k_t (n values) and v_t (m values) are columns of a row buffer x (T, ld), float32 or bfloat16: q of head h at
// [oq + (h / rep) n, ...), k at [ok + (h / rep) n, ...) (rep = H / qk_heads heads share one q and k), v at [ov + h m, ...).
// The decays are float32 rows (T, lda): a_t of head h at [oa + h] or, per channel, at [oa + h n, ...); beta_t float32 at
// [ob + h] of rows (T, ldb).  Nothing is rounded below float32 between the rows and the output (T, H m).
//
// gated_state_scan: one block per (sequence, head, tile of 16 value columns).  Thread (rg, jl) = (tid & 15, tid >> 4)
// holds the state's rows rg, rg + 16, ... of column jl in registers; the sixteen partial sums of a column (S^T k, S^T q)
// are neighbours in a wavefront and are added by moves between lanes.  A step's tokens come through LDS sixteen (wide
// keys: eight) at a time, the next batch asked for while this one is computed.  Every sum runs in one fixed order,
// whatever the step's cut: a sequence fed whole, in portions or token by token leaves the same state and outputs, bit
// for bit.  A step of single tokens is the same kernel with one token a block.
//
// Long portions, segment by segment.  Over a run of tokens the state goes S -> M S + B with an n x n matrix M (what the
// decays and the delta rule's corrections do to a state, whatever it holds) and B (what the run writes, starting from
// nothing).  So the segments of a long portion run side by side: the same kernel gives every segment's B (from a state
// of zeros) and M (from the identity, with every value zero), gated_state_chain walks a sequence's segments in order
// (S_(s+1) = M_s S_s + B_s, a product of n x n by n x 16 a block and segment) and leaves every segment's first state,
// and the kernel runs once more from those states for the outputs.  The same arithmetic in another association.
//
// delta_rule_prep: what the gated delta rule computes between its convolutions and the recurrence, in float32:
//   q <- q / sqrt(sum q^2 + unit_eps) * q_scale,  k <- k / sqrt(sum k^2 + unit_eps)        per (token, q/k head), in place
//   g = exp(-exp(A_log[h]) softplus(a + dt_bias[h])),  beta = sigmoid(b)                     per (token, head)
// channel_decay: alpha = sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau), elementwise in place.
#include "common.h"

#define GR_RG 16          // lanes that share a state column (each holds every sixteenth row of it)
#define GR_COLS 16        // value columns a block (256 threads / GR_RG)

__device__ __forceinline__ float gr_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// The sum over the sixteen neighbouring lanes that share a column (a row of lanes): moves within quads, then the
// mirrors of eight and of sixteen lanes (lane i <-> 7 - i, then i <-> 15 - i, which lie in parts not yet added); no trip
// through LDS.  Every lane gets the sum; its order is fixed.
__device__ __forceinline__ float gr_sum16(float x) {
  x += dpp_move<0xB1>(x);    // quad_perm [1,0,3,2]
  x += dpp_move<0x4E>(x);    // quad_perm [2,3,0,1]
  x += dpp_move<0x141>(x);   // row_half_mirror
  x += dpp_move<0x140>(x);   // row_mirror
  return x;
}

// RMAX: state rows a thread (keys up to 16 RMAX wide).  A thread's rows i = rg + 16 r lie side by side in LDS (place
// rg RMAX + r), so that it reads them up to sixteen bytes at a time; the places of rows beyond n hold zeros.  The tokens of the next batch are asked for before this
// batch is computed and land in registers meanwhile.
template <typename TI, int RMAX, bool VEC, bool DELTA>
__global__ void __launch_bounds__(256)
gated_state_scan_kernel(const TI* __restrict__ x, int ld, int oq, int ok, int ov, int rep, float q_scale,
                        const float* __restrict__ decay, int lda, int oa, const float* __restrict__ beta, int ldb,
                        int ob, float* __restrict__ state, const int* __restrict__ q_start,
                        const int* __restrict__ slots, float* __restrict__ out, int H, int n, int m) {
  constexpr int NMAX = GR_RG * RMAX;
  constexpr int TB = NMAX <= 128 ? 16 : 8;                 // tokens staged at once
  constexpr int PER = (TB * NMAX + 255) / 256;             // values of q (k, decays) a thread stages
  constexpr int PERV = (TB * GR_COLS + 255) / 256;
  __shared__ __attribute__((aligned(16))) float qs[TB][NMAX];
  __shared__ __attribute__((aligned(16))) float ks[TB][NMAX];
  __shared__ __attribute__((aligned(16))) float al[VEC ? TB : 1][VEC ? NMAX : 4];
  __shared__ float vs[TB][GR_COLS];
  __shared__ float a1[TB], bs[TB];
  const int seq = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * GR_COLS;
  const int tid = threadIdx.x, rg = tid & (GR_RG - 1), jl = tid / GR_RG, j = j0 + jl;
  const int t0 = q_start[seq], t1 = q_start[seq + 1];
  if (t1 <= t0) return;
  const int hq = h / rep;
  float* S = state + (((size_t)slots[seq] * H + h) * n) * m;
  float s[RMAX];
#pragma unroll
  for (int r = 0; r < RMAX; ++r) {
    const int i = rg + GR_RG * r;
    s[r] = (i < n && j < m) ? S[(size_t)i * m + j] : 0.f;
  }
  // a batch's values on their way: asked for one batch ahead, kept in registers until the batch before has been read
  float rq[PER], rk[PER], ra[VEC ? PER : 1], rv[PERV], r1 = 0.f, rb = 0.f;
  auto ask = [&](int tb) {
    const int nb = t1 - tb < TB ? t1 - tb : TB;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int idx = tid + u * 256;
      const int tt = idx / n, i = idx - tt * n;
      const bool live = idx < nb * n;
      const TI* row = x + (size_t)(tb + (live ? tt : 0)) * ld;
      rq[u] = live ? to_f32(row[oq + hq * n + i]) * q_scale : 0.f;
      rk[u] = live ? to_f32(row[ok + hq * n + i]) : 0.f;
      if (VEC) ra[u] = live ? decay[(size_t)(tb + tt) * lda + oa + h * n + i] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < PERV; ++u) {
      const int idx = tid + u * 256;
      const int tt = idx / GR_COLS, c = idx - tt * GR_COLS;
      rv[u] = (ov >= 0 && idx < nb * GR_COLS && j0 + c < m) ? to_f32(x[(size_t)(tb + tt) * ld + ov + h * m + j0 + c]) : 0.f;
    }
    if (tid < nb) {
      if (!VEC) r1 = decay[(size_t)(tb + tid) * lda + oa + h];
      if (DELTA) rb = beta[(size_t)(tb + tid) * ldb + ob + h];
    }
  };
  auto put = [&](int tb) {
    const int nb = t1 - tb < TB ? t1 - tb : TB;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int idx = tid + u * 256;
      if (idx < nb * n) {
        const int tt = idx / n, i = idx - tt * n;
        const int place = (i & (GR_RG - 1)) * RMAX + (i >> 4);
        qs[tt][place] = rq[u];
        ks[tt][place] = rk[u];
        if (VEC) al[tt][place] = ra[u];
      }
    }
#pragma unroll
    for (int u = 0; u < PERV; ++u) {
      const int idx = tid + u * 256;
      if (idx < nb * GR_COLS) vs[idx / GR_COLS][idx % GR_COLS] = rv[u];
    }
    if (tid < nb) {
      if (!VEC) a1[tid] = r1;
      if (DELTA) bs[tid] = rb;
    }
  };
  // the places of rows beyond n (where n is no multiple of 16) are written here once and never again: such a row of
  // the state starts at zero and stays there, whatever stands beside it
  for (int idx = tid; idx < TB * NMAX; idx += 256) {
    qs[idx / NMAX][idx % NMAX] = 0.f;
    ks[idx / NMAX][idx % NMAX] = 0.f;
    if (VEC) al[idx / NMAX][idx % NMAX] = 0.f;
  }
  struct Tok {
    float k[RMAX], q[RMAX], a[VEC ? RMAX : 1];
    float v, a1, b;
  };
  auto take = [&](Tok& t, int tt) __attribute__((always_inline)) {
    const float* kr = &ks[tt][rg * RMAX];
    const float* qr = &qs[tt][rg * RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      t.k[r] = kr[r];
      t.q[r] = qr[r];
      if (VEC) t.a[r] = al[tt][rg * RMAX + r];
    }
    t.v = vs[tt][jl];
    t.a1 = VEC ? 0.f : a1[tt];
    t.b = DELTA ? bs[tt] : 0.f;
  };
  auto advance = [&](const Tok& t, int row) __attribute__((always_inline)) {
    float u = t.v;
    float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      s[r] *= VEC ? t.a[r] : t.a1;
      if (DELTA) {
        const float w = s[r] * t.k[r];
        if ((r & 3) == 0) p0 += w; else if ((r & 3) == 1) p1 += w; else if ((r & 3) == 2) p2 += w; else p3 += w;
      }
    }
    if (DELTA) u = t.b * (u - gr_sum16((p0 + p1) + (p2 + p3)));
    p0 = p1 = p2 = p3 = 0.f;
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      s[r] = fmaf(t.k[r], u, s[r]);
      const float w = s[r] * t.q[r];
      if ((r & 3) == 0) p0 += w; else if ((r & 3) == 1) p1 += w; else if ((r & 3) == 2) p2 += w; else p3 += w;
    }
    const float part = gr_sum16((p0 + p1) + (p2 + p3));
    if (out && rg == 0 && j < m) out[((size_t)row * H + h) * m + j] = part;
  };
  ask(t0);
  for (int tb = t0; tb < t1; tb += TB) {
    const int nb = t1 - tb < TB ? t1 - tb : TB;
    __syncthreads();                                   // the batch before has been read
    put(tb);
    __syncthreads();
    if (tb + TB < t1) ask(tb + TB);
    // A token's operands come from LDS one token ahead (two sets of registers, used in turn), so that their way from
    // LDS lies behind the token before; the chain from state to state is all that a token waits for.
    Tok ta, tb2;
    take(ta, 0);
    for (int tt = 0; tt < nb; tt += 2) {
      if (tt + 1 < nb) take(tb2, tt + 1);
      advance(ta, tb + tt);
      if (tt + 1 < nb) {
        if (tt + 2 < nb) take(ta, tt + 2);
        advance(tb2, tb + tt + 1);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RMAX; ++r) {
    const int i = rg + GR_RG * r;
    if (i < n && j < m) S[(size_t)i * m + j] = s[r];
  }
}

extern "C" int gs_gated_state_scan(const void* x, int dtype, int ld, int oq, int ok, int ov, int qk_heads, float q_scale,
                                   const float* decay, int lda, int oa, int per_channel, const float* beta, int ldb,
                                   int ob, float* state, const int* q_start, const int* slots, float* out, int nseq,
                                   int H, int n, int m, hipStream_t stream) {
  GS_REQUIRE(nseq >= 0 && H > 0 && n > 0 && m > 0, "gated_state_scan: bad sizes nseq=%d H=%d n=%d m=%d", nseq, H, n, m);
  GS_REQUIRE(n <= 256, "gated_state_scan: keys of %d features, the kernel holds up to 256", n);
  GS_REQUIRE(qk_heads > 0 && H % qk_heads == 0, "gated_state_scan: %d heads do not share %d queries and keys evenly", H,
             qk_heads);
  GS_REQUIRE(H <= 65535 && (m + GR_COLS - 1) / GR_COLS <= 65535, "gated_state_scan: too many heads or value columns");
  // (ov < 0: every value is zero, what the state does to itself over the tokens; out null: the states alone are wanted)
  GS_REQUIRE(oq >= 0 && ok >= 0 && oq + qk_heads * n <= ld && ok + qk_heads * n <= ld && (ov < 0 || ov + H * m <= ld),
             "gated_state_scan: q, k or v lie outside the rows of %d", ld);
  GS_REQUIRE(decay && oa >= 0 && oa + (per_channel ? H * n : H) <= lda, "gated_state_scan: the decays lie outside their rows of %d", lda);
  GS_REQUIRE(!beta || (ob >= 0 && ob + H <= ldb), "gated_state_scan: the write strengths lie outside their rows of %d", ldb);
  if (nseq == 0) return 0;
  dim3 grid(nseq, H, (m + GR_COLS - 1) / GR_COLS);
  const int rep = H / qk_heads;
#define GR_RUN(TI, R, V, D)                                                                                         \
  gated_state_scan_kernel<TI, R, V, D><<<grid, 256, 0, stream>>>((const TI*)x, ld, oq, ok, ov, rep, q_scale, decay, \
                                                                 lda, oa, beta, ldb, ob, state, q_start, slots, out, H, n, m)
#define GR_RUN_R(TI, V, D)                   \
  if (n <= 32) GR_RUN(TI, 2, V, D);          \
  else if (n <= 64) GR_RUN(TI, 4, V, D);     \
  else if (n <= 128) GR_RUN(TI, 8, V, D);    \
  else GR_RUN(TI, 16, V, D)
#define GR_RUN_T(TI)                                      \
  if (per_channel && beta) { GR_RUN_R(TI, true, true); }  \
  else if (per_channel) { GR_RUN_R(TI, true, false); }    \
  else if (beta) { GR_RUN_R(TI, false, true); }           \
  else { GR_RUN_R(TI, false, false); }
  if (dtype == GS_F32) {
    GR_RUN_T(float)
  } else if (dtype == GS_BF16) {
    GR_RUN_T(bf16)
  } else {
    GS_REQUIRE(false, "gated_state_scan: unknown dtype %d", dtype);
  }
#undef GR_RUN_T
#undef GR_RUN_R
#undef GR_RUN
  GS_LAUNCH_CHECK("gated_state_scan");
  return 0;
}

// One block per (sequence, head, 16 value columns): S (n x 16) in LDS; for the sequence's segments in order, the state a
// segment starts from goes to `first`, then S <- M_seg S + B_seg; the last state is the request's.  M (segments, H, n, n),
// B and first (segments, H, n, m), state (slots, H, n, m); seq_seg (nseq + 1): where each sequence's segments begin.
// M comes through LDS in tiles of R rows (R n <= 4096 values, R a multiple of 16 or n itself), read with 16-byte loads
// one tile ahead of the products that use it (the walk is a chain of small steps: what it waits for is memory), and so
// do the rows of B.
#define GR_CHAIN_TILE 4096
__global__ void __launch_bounds__(256)
gated_state_chain_kernel(const float* __restrict__ M, const float* __restrict__ B, float* __restrict__ first,
                         float* __restrict__ state, const int* __restrict__ seq_seg, const int* __restrict__ slots, int H,
                         int n, int m, int R) {
  extern __shared__ float ch_s[];             // S and its successor, n x 16 each; then a tile of M, R x n
  float* S = ch_s;
  float* N = ch_s + (size_t)n * GR_COLS;
  float* Mt = ch_s + 2 * (size_t)n * GR_COLS;
  const int seq = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * GR_COLS;
  const int tid = threadIdx.x, jl = tid & (GR_COLS - 1), rl = tid / GR_COLS, j = j0 + jl;
  const int s0 = seq_seg[seq], s1 = seq_seg[seq + 1];
  if (s1 <= s0) return;
  float* own = state + (((size_t)slots[seq] * H + h) * n) * m;
  for (int i = rl; i < n; i += 16) S[i * GR_COLS + jl] = j < m ? own[(size_t)i * m + j] : 0.f;
  const int tps = (n + R - 1) / R, total = (s1 - s0) * tps;      // tiles a segment, tiles in all
  const bool vec = (n & 3) == 0;                                   // (rows of M start at multiples of 16 bytes)
  float pm[16], pb[4];
  auto ask = [&](int t) {
    const int sg = s0 + t / tps, r0 = (t % tps) * R;
    const int len = (r0 + R < n ? R : n - r0) * n;
    const float* src = M + (((size_t)sg * H + h) * n + r0) * n;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int at = (tid + 256 * u) * 4;
      if (vec && at + 3 < len) {
        const float4 v = *reinterpret_cast<const float4*>(src + at);
        pm[4 * u] = v.x; pm[4 * u + 1] = v.y; pm[4 * u + 2] = v.z; pm[4 * u + 3] = v.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) pm[4 * u + e] = at + e < len ? src[at + e] : 0.f;
      }
    }
    const float* bsrc = B + ((size_t)sg * H + h) * n * m;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = r0 + rl + 16 * r;
      pb[r] = (rl + 16 * r < R && i < n && j < m) ? bsrc[(size_t)i * m + j] : 0.f;
    }
  };
  ask(0);
  for (int t = 0; t < total; ++t) {
    const int sg = s0 + t / tps, r0 = (t % tps) * R;
    __syncthreads();                          // the tile before has been read (and, at a segment's start, S is whole)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int at = (tid + 256 * u) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (at + e < R * n) Mt[at + e] = pm[4 * u + e];
    }
    float bv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) bv[r] = pb[r];
    __syncthreads();
    if (t + 1 < total) ask(t + 1);
    if (r0 == 0) {
      float* Fs = first + ((size_t)sg * H + h) * n * m;
      for (int i = rl; i < n; i += 16)
        if (j < m) Fs[(size_t)i * m + j] = S[i * GR_COLS + jl];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int ir = rl + 16 * r, i = r0 + ir;
      if (ir < R && i < n) {
        const float* row = Mt + (size_t)ir * n;
        float a0 = bv[r], a1 = 0.f, a2 = 0.f, a3 = 0.f;
        int k = 0;
        for (; k + 3 < n; k += 4) {
          a0 = fmaf(row[k], S[k * GR_COLS + jl], a0);
          a1 = fmaf(row[k + 1], S[(k + 1) * GR_COLS + jl], a1);
          a2 = fmaf(row[k + 2], S[(k + 2) * GR_COLS + jl], a2);
          a3 = fmaf(row[k + 3], S[(k + 3) * GR_COLS + jl], a3);
        }
        for (; k < n; ++k) a0 = fmaf(row[k], S[k * GR_COLS + jl], a0);
        N[i * GR_COLS + jl] = (a0 + a1) + (a2 + a3);
      }
    }
    if (r0 + R >= n) {                         // the segment's last tile: its successor is whole
      __syncthreads();
      float* x = S;
      S = N;
      N = x;
    }
  }
  __syncthreads();
  for (int i = rl; i < n; i += 16)
    if (j < m) own[(size_t)i * m + j] = S[i * GR_COLS + jl];
}

extern "C" int gs_gated_state_chain(const float* M, const float* B, float* first, float* state, const int* seq_seg,
                                    const int* slots, int nseq, int H, int n, int m, hipStream_t stream) {
  GS_REQUIRE(nseq >= 0 && H > 0 && n > 0 && n <= 256 && m > 0, "gated_state_chain: bad sizes nseq=%d H=%d n=%d m=%d", nseq, H, n, m);
  GS_REQUIRE(H <= 65535 && (m + GR_COLS - 1) / GR_COLS <= 65535, "gated_state_chain: too many heads or value columns");
  if (nseq == 0) return 0;
  // rows of M a tile: all of them where n x n values fit, else as many whole sixteens as do (n <= 256: at least 16)
  int R = n * n <= GR_CHAIN_TILE ? n : (GR_CHAIN_TILE / n) / 16 * 16;
  if (R > 64) R = 64;                          // (a thread keeps four rows of B for a tile)
  dim3 grid(nseq, H, (m + GR_COLS - 1) / GR_COLS);
  const size_t lds = (2 * (size_t)n * GR_COLS + (size_t)R * n) * sizeof(float);
  gated_state_chain_kernel<<<grid, 256, lds, stream>>>(M, B, first, state, seq_seg, slots, H, n, m, R);
  GS_LAUNCH_CHECK("gated_state_chain");
  return 0;
}

// One block of 256 threads per token: a wavefront per q or k head in turn, then the heads' gates.
//   c (T, ldc) float32: q heads at [0, G n), k heads at [G n, 2 G n), normed in place
//   rows (T, ldr): the decay's product at [oa + h], the write strength's at [obeta + h]
//   gates (T, 2 H) float32: g at [h], beta at [H + h]
template <typename TR>
__global__ void __launch_bounds__(256)
delta_rule_prep_kernel(float* __restrict__ c, int ldc, int G, int n, float q_scale, float unit_eps,
                       const TR* __restrict__ rows, int ldr, int oa, int obeta, const float* __restrict__ a_log,
                       const float* __restrict__ dt_bias, float* __restrict__ gates, int H) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int u = wave; u < 2 * G; u += 4) {
    float* v = c + (size_t)t * ldc + (size_t)u * n;
    float ss = 0.f;
    for (int i = lane; i < n; i += 64) ss += v[i] * v[i];
    ss = wave_sum(ss);
    const float inv = (u < G ? q_scale : 1.f) / sqrtf(ss + unit_eps);
    for (int i = lane; i < n; i += 64) v[i] *= inv;
  }
  for (int h = threadIdx.x; h < H; h += 256) {
    const float a = to_f32(rows[(size_t)t * ldr + oa + h]), b = to_f32(rows[(size_t)t * ldr + obeta + h]);
    gates[(size_t)t * 2 * H + h] = expf(-expf(a_log[h]) * gr_softplus(a + dt_bias[h]));
    gates[(size_t)t * 2 * H + H + h] = 1.f / (1.f + expf(-b));
  }
}

extern "C" int gs_delta_rule_prep(float* c, int ldc, int G, int n, float q_scale, float unit_eps, const void* rows,
                                  int rows_dtype, int ldr, int oa, int obeta, const float* a_log, const float* dt_bias,
                                  float* gates, int T, int H, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && G > 0 && n > 0 && H > 0 && 2 * G * n <= ldc, "delta_rule_prep: bad sizes T=%d G=%d n=%d H=%d ldc=%d",
             T, G, n, H, ldc);
  GS_REQUIRE(oa >= 0 && obeta >= 0 && oa + H <= ldr && obeta + H <= ldr, "delta_rule_prep: the gates' products lie outside the rows of %d", ldr);
  GS_REQUIRE(unit_eps >= 0.f, "delta_rule_prep: bad eps");
  if (T == 0) return 0;
  if (rows_dtype == GS_F32)
    delta_rule_prep_kernel<float><<<T, 256, 0, stream>>>(c, ldc, G, n, q_scale, unit_eps, (const float*)rows, ldr, oa,
                                                          obeta, a_log, dt_bias, gates, H);
  else if (rows_dtype == GS_BF16)
    delta_rule_prep_kernel<bf16><<<T, 256, 0, stream>>>(c, ldc, G, n, q_scale, unit_eps, (const bf16*)rows, ldr, oa,
                                                         obeta, a_log, dt_bias, gates, H);
  else
    GS_REQUIRE(false, "delta_rule_prep: unknown dtype %d", rows_dtype);
  GS_LAUNCH_CHECK("delta_rule_prep");
  return 0;
}

__global__ void channel_decay_kernel(float* __restrict__ z, long total, float inv_tau) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) z[i] = expf(-gr_softplus(-z[i]) * inv_tau);
}

extern "C" int gs_channel_decay(float* z, long total, float tau, hipStream_t stream) {
  GS_REQUIRE(total >= 0 && tau > 0.f, "channel_decay: bad sizes or tau");
  if (total == 0) return 0;
  channel_decay_kernel<<<gs_ceil_div(total, 256), 256, 0, stream>>>(z, total, 1.f / tau);
  GS_LAUNCH_CHECK("channel_decay");
  return 0;
}
