// Attention through a cached latent row: the kernels around the products, and the general attention kernel.
//
// A token's cache row is [z | k_rot]: z = the normed key/value latent (c numbers), k_rot = the rotated key features
// that all heads share (r numbers).  Head h's key is (W_uk[h] z | k_rot) and its value W_uv[h] z, so with
// q~ = (W_uk[h]^T q_plain | q_rot) the score is q~ . [z | k_rot] and the head's output W_uv[h] (sum_j p_j z_j):
// every head attends over the same rows (one key head of width c + r whose first c columns are also its values),
// and neither keys nor values of single heads are ever formed.
//
//   latent_prep       per token: RMS norm of the query latent -> rows for the query product; RMS norm of the
//                     key/value latent, rotation of the shared key features, both into the token's cache row
//   latent_q_rot      rotates the rotated part of every head's query into its place behind the absorbed part
//   heads_product     Y[t, h, :] = W[h] X[t, h, :] for all heads in one launch, with an optional gate: times
//                     sigmoid(G[t, h]), or times sigmoid(G[t, h N + n]) for output n (a gate each); float32 FMAs in a
//                     fixed summation order, or the matrix cores for bfloat16
//   attention_latent  the general attention kernel over such rows: any sizes, float32 arithmetic
//
// All norms, angles, scores, softmax weights and the gate's sigmoid are float32.
#include "common.h"

template <typename T>
__global__ void latent_prep_kernel(const T* __restrict__ down, int ld, int q_off, int q_rank, int kv_off, int c, int r,
                                   const float* __restrict__ qw, const float* __restrict__ kvw, float eps,
                                   const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                   const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                   const int* __restrict__ block_table, int max_blocks, int page_size,
                                   T* __restrict__ cache, T* __restrict__ a_out, int write_kv) {
  __shared__ float red[17];
  const int t = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  const T* row = down + (size_t)t * ld;
  float ss = 0.f;
  for (int j = tid; j < q_rank; j += nt) {
    const float v = to_f32(row[q_off + j]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  float inv = norm_inverse(ss, (float)q_rank, eps);
  for (int j = tid; j < q_rank; j += nt)
    a_out[(size_t)t * q_rank + j] = from_f32<T>(to_f32(row[q_off + j]) * inv * qw[j]);
  if (!write_kv) return;
  ss = 0.f;
  for (int j = tid; j < c; j += nt) {
    const float v = to_f32(row[kv_off + j]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  inv = norm_inverse(ss, (float)c, eps);
  const int pos = positions[t];
  const int page = block_table[(size_t)seq_of_token[t] * max_blocks + pos / page_size];
  T* dst = cache + ((size_t)page * page_size + pos % page_size) * (size_t)(c + r);
  for (int j = tid; j < c; j += nt) dst[j] = from_f32<T>(to_f32(row[kv_off + j]) * inv * kvw[j]);
  const int half = r / 2;
  for (int j = tid; j < half; j += nt) {
    const float u = to_f32(row[kv_off + c + j]), v = to_f32(row[kv_off + c + j + half]);
    const float cs = cos_t[(size_t)pos * half + j], sn = sin_t[(size_t)pos * half + j];
    dst[c + j] = from_f32<T>(u * cs - v * sn);
    dst[c + j + half] = from_f32<T>(v * cs + u * sn);
  }
}

extern "C" int gs_latent_prep(const void* down, int dtype, int ld, int q_off, int q_rank, int kv_off, int c, int r,
                              const float* qw, const float* kvw, float eps, const float* cos_t, const float* sin_t,
                              const int* positions, const int* seq_of_token, const int* block_table, int max_blocks,
                              int page_size, void* cache, void* a_out, int write_kv, int ntok, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && q_rank > 0 && c > 0 && r >= 0 && r % 2 == 0, "latent_prep: bad sizes T=%d q_rank=%d c=%d r=%d",
             ntok, q_rank, c, r);
  GS_REQUIRE(q_off >= 0 && kv_off >= 0 && q_off + q_rank <= ld && kv_off + c + r <= ld,
             "latent_prep: columns %d+%d, %d+%d+%d outside rows of %d", q_off, q_rank, kv_off, c, r, ld);
  GS_REQUIRE(page_size > 0 && max_blocks > 0, "latent_prep: bad page_size/max_blocks");
  if (ntok == 0) return 0;
  if (dtype == GS_F32)
    latent_prep_kernel<float><<<ntok, 256, 0, stream>>>((const float*)down, ld, q_off, q_rank, kv_off, c, r, qw, kvw, eps,
                                                        cos_t, sin_t, positions, seq_of_token, block_table, max_blocks,
                                                        page_size, (float*)cache, (float*)a_out, write_kv);
  else if (dtype == GS_BF16)
    latent_prep_kernel<bf16><<<ntok, 256, 0, stream>>>((const bf16*)down, ld, q_off, q_rank, kv_off, c, r, qw, kvw, eps,
                                                       cos_t, sin_t, positions, seq_of_token, block_table, max_blocks,
                                                       page_size, (bf16*)cache, (bf16*)a_out, write_kv);
  else
    GS_REQUIRE(false, "latent_prep: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("latent_prep");
  return 0;
}

// q (T, ldq): head h at [h (n + r), ...), its last r columns rotated into qa (T, H (c + r)) at [h (c + r) + c, ...).
template <typename T>
__global__ void latent_q_rot_kernel(const T* __restrict__ q, int ldq, int H, int n, int r, int c,
                                    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                    const int* __restrict__ positions, T* __restrict__ qa) {
  const int t = blockIdx.x, half = r / 2, pos = positions[t];
  const T* row = q + (size_t)t * ldq;
  T* dst = qa + (size_t)t * H * (c + r);
  for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
    const int h = idx / half, j = idx % half;
    const float u = to_f32(row[h * (n + r) + n + j]), v = to_f32(row[h * (n + r) + n + j + half]);
    const float cs = cos_t[(size_t)pos * half + j], sn = sin_t[(size_t)pos * half + j];
    dst[h * (c + r) + c + j] = from_f32<T>(u * cs - v * sn);
    dst[h * (c + r) + c + j + half] = from_f32<T>(v * cs + u * sn);
  }
}

extern "C" int gs_latent_q_rot(const void* q, int dtype, int ldq, int H, int n, int r, int c, const float* cos_t,
                               const float* sin_t, const int* positions, void* qa, int ntok, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && H > 0 && n >= 0 && r >= 0 && r % 2 == 0 && c > 0, "latent_q_rot: bad sizes");
  GS_REQUIRE(ldq >= H * (n + r), "latent_q_rot: rows of %d hold no %d heads of %d", ldq, H, n + r);
  if (ntok == 0 || r == 0) return 0;
  if (dtype == GS_F32)
    latent_q_rot_kernel<float><<<ntok, 128, 0, stream>>>((const float*)q, ldq, H, n, r, c, cos_t, sin_t, positions,
                                                         (float*)qa);
  else if (dtype == GS_BF16)
    latent_q_rot_kernel<bf16><<<ntok, 128, 0, stream>>>((const bf16*)q, ldq, H, n, r, c, cos_t, sin_t, positions,
                                                        (bf16*)qa);
  else
    GS_REQUIRE(false, "latent_q_rot: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("latent_q_rot");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Y[m, h, :N] = W[h] (N, K) . X[m, h, :K], all heads in one launch: head h's rows of X start hx elements after head
// h - 1's, those of Y hy elements.  The summation order of an output is that of the plain tiled product (chunks of 64
// from zero in ascending k, then the chunks' sums), so a value depends neither on M nor on its neighbours.
#define HP_TM 64
#define HP_TN 64
#define HP_TK 16

template <typename TX, typename TW>
__global__ void heads_product_kernel(const TX* __restrict__ X, int ldx, int hx, const TW* __restrict__ W,
                                     TX* __restrict__ Y, int ldy, int hy, const TX* __restrict__ G, int ldg,
                                     int gate_each, int M, int N, int K) {
  __shared__ float xs[HP_TK][HP_TM + 4];
  __shared__ float ws[HP_TK][HP_TN + 4];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int h = blockIdx.z, m0 = blockIdx.y * HP_TM, n0 = blockIdx.x * HP_TN;
  X += (size_t)h * hx;
  Y += (size_t)h * hy;
  W += (size_t)h * N * K;
  float acc[4][4], tot[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = tot[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += HP_TK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256, r = idx >> 4, kk = idx & 15;
      const int m = m0 + r, n = n0 + r, k = k0 + kk;
      xs[kk][r] = (m < M && k < K) ? to_f32(X[(size_t)m * ldx + k]) : 0.f;
      ws[kk][r] = (n < N && k < K) ? to_f32(W[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HP_TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
    if (((k0 / HP_TK) & (GS_SUM_CHUNK / HP_TK - 1)) == GS_SUM_CHUNK / HP_TK - 1 || k0 + HP_TK >= K) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tot[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
    float gate = 1.f;
    if (G && !gate_each) gate = 1.f / (1.f + expf(-to_f32(G[(size_t)m * ldg + h])));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      if (G && gate_each) gate = 1.f / (1.f + expf(-to_f32(G[(size_t)m * ldg + (size_t)h * N + n])));
      Y[(size_t)m * ldy + n] = from_f32<TX>(tot[i][j] * gate);
    }
  }
}

// The same product on the matrix cores (bfloat16 rows and weights, float32 sums): v_mfma_f32_16x16x32_bf16 with both
// operands loaded straight from memory in operand order (lane l: row or weight row l % 16, eight consecutive k at
// 8 (l / 16)); a head's weight is small and stays in the caches, so nothing is staged.  A wavefront owns 16 MTW rows x
// 16 NTW columns of one head; the four wavefronts of a block own four such pieces, and no barrier is needed.
typedef __attribute__((ext_vector_type(8))) __bf16 hp_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float hp_f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned hp_u32x4_t;

template <int NTW, int MTW>
__global__ __launch_bounds__(256) void heads_product_mfma_kernel(const bf16* __restrict__ X, int ldx, int hx,
                                                                 const bf16* __restrict__ W, bf16* __restrict__ Y,
                                                                 int ldy, int hy, const bf16* __restrict__ G, int ldg,
                                                                 int gate_each, int M, int N, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
  const int h = blockIdx.y;
  const int mtiles = (M + 16 * MTW - 1) / (16 * MTW), ngroups = (N + 16 * NTW - 1) / (16 * NTW);
  const int item = blockIdx.x * 4 + wave;
  if (item >= mtiles * ngroups) return;
  const int m0 = (item % mtiles) * 16 * MTW, n0 = (item / mtiles) * 16 * NTW;
  const bf16* xp[MTW];
#pragma unroll
  for (int i = 0; i < MTW; ++i) {
    const int mrow = m0 + 16 * i + r16 < M ? m0 + 16 * i + r16 : M - 1;
    xp[i] = X + (size_t)mrow * ldx + (size_t)h * hx + 8 * g;
  }
  const bf16* wp[NTW];
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    const int n = n0 + 16 * j + r16 < N ? n0 + 16 * j + r16 : N - 1;
    wp[j] = W + ((size_t)h * N + n) * K + 8 * g;
  }
  hp_f32x4_t acc[MTW][NTW];
#pragma unroll
  for (int i = 0; i < MTW; ++i)
#pragma unroll
    for (int j = 0; j < NTW; ++j) acc[i][j] = hp_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool in = k0 + 8 * g < K;                      // K in whole pieces of 8: a piece is inside or outside
    const int kk = in ? k0 : -8 * g;
    hp_u32x4_t a[MTW];
#pragma unroll
    for (int i = 0; i < MTW; ++i) {
      a[i] = *reinterpret_cast<const hp_u32x4_t*>(xp[i] + kk);
      a[i] = in ? a[i] : hp_u32x4_t{0u, 0u, 0u, 0u};
    }
    hp_u32x4_t b[NTW];
#pragma unroll
    for (int j = 0; j < NTW; ++j) {
      b[j] = *reinterpret_cast<const hp_u32x4_t*>(wp[j] + kk);
      b[j] = in ? b[j] : hp_u32x4_t{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < MTW; ++i)
#pragma unroll
      for (int j = 0; j < NTW; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(hp_bf16x8_t, a[i]),
                                                            __builtin_bit_cast(hp_bf16x8_t, b[j]), acc[i][j], 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < MTW; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int m = m0 + 16 * i + 4 * g + e;
      if (m >= M) continue;
      float gate = 1.f;
      if (G && !gate_each) gate = 1.f / (1.f + expf(-to_f32(G[(size_t)m * ldg + h])));
#pragma unroll
      for (int j = 0; j < NTW; ++j) {
        const int n = n0 + 16 * j + r16;
        if (n >= N) continue;
        if (G && gate_each) gate = 1.f / (1.f + expf(-to_f32(G[(size_t)m * ldg + (size_t)h * N + n])));
        Y[(size_t)m * ldy + (size_t)h * hy + n] = f32_to_bf16(acc[i][j][e] * gate);
      }
    }
}

extern "C" int gs_heads_product(const void* X, int x_dtype, int ldx, int hx, const void* W, int w_dtype, void* Y,
                                int ldy, int hy, const void* G, int ldg, int gate_each, int M, int N, int K, int H,
                                hipStream_t stream) {
  GS_REQUIRE(M >= 0 && N > 0 && K > 0 && H > 0, "heads_product: bad sizes M=%d N=%d K=%d H=%d", M, N, K, H);
  GS_REQUIRE(H <= 65535 && gs_ceil_div(M, HP_TM) <= 65535, "heads_product: too many heads or rows for one launch");
  GS_REQUIRE((long)(H - 1) * hx + K <= ldx && (long)(H - 1) * hy + N <= ldy,
             "heads_product: heads reach past their rows (ldx=%d hx=%d K=%d, ldy=%d hy=%d N=%d)", ldx, hx, K, ldy, hy, N);
  GS_REQUIRE(G == nullptr || ldg >= (gate_each ? H * N : H), "heads_product: gate rows of %d hold no gates for %d heads", ldg, H);
  if (M == 0) return 0;
  if (x_dtype == GS_BF16 && w_dtype == GS_BF16 && K % 8 == 0 && ldx % 8 == 0 && hx % 8 == 0 && ((uintptr_t)X & 15) == 0 &&
      ((uintptr_t)W & 15) == 0) {
    // few rows: narrow pieces, so that a head's weight is spread over more wavefronts; many: 32 x 64 a wavefront
    const int ntw = M <= 64 ? 1 : 4, mtw = M <= 64 ? 1 : 2;
    const int mtiles = gs_ceil_div(M, 16 * mtw);
    const long items = (long)mtiles * gs_ceil_div(N, 16 * ntw);
    GS_REQUIRE(items / 4 + 1 < (1L << 31), "heads_product: too many tiles");
    dim3 grid((unsigned)gs_ceil_div(items, 4), H);
    if (ntw == 1)
      heads_product_mfma_kernel<1, 1><<<grid, 256, 0, stream>>>((const bf16*)X, ldx, hx, (const bf16*)W, (bf16*)Y, ldy, hy,
                                                            (const bf16*)G, ldg, gate_each, M, N, K);
    else
      heads_product_mfma_kernel<4, 2><<<grid, 256, 0, stream>>>((const bf16*)X, ldx, hx, (const bf16*)W, (bf16*)Y, ldy, hy,
                                                            (const bf16*)G, ldg, gate_each, M, N, K);
    GS_LAUNCH_CHECK("heads_product_mfma");
    return 0;
  }
  dim3 grid(gs_ceil_div(N, HP_TN), gs_ceil_div(M, HP_TM), H);
  if (x_dtype == GS_F32 && w_dtype == GS_F32)
    heads_product_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)X, ldx, hx, (const float*)W, (float*)Y,
                                                                 ldy, hy, (const float*)G, ldg, gate_each, M, N, K);
  else if (x_dtype == GS_BF16 && w_dtype == GS_BF16)
    heads_product_kernel<bf16, bf16><<<grid, 256, 0, stream>>>((const bf16*)X, ldx, hx, (const bf16*)W, (bf16*)Y, ldy,
                                                               hy, (const bf16*)G, ldg, gate_each, M, N, K);
  else if (x_dtype == GS_BF16 && w_dtype == GS_F32)
    heads_product_kernel<bf16, float><<<grid, 256, 0, stream>>>((const bf16*)X, ldx, hx, (const float*)W, (bf16*)Y, ldy,
                                                                hy, (const bf16*)G, ldg, gate_each, M, N, K);
  else
    GS_REQUIRE(false, "heads_product: unsupported types %d %d", x_dtype, w_dtype);
  GS_LAUNCH_CHECK("heads_product");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// The general attention kernel over latent rows: one wavefront per (query token, head).  The query at position p of
// its sequence sees the rows lo..p, lo = 0 or p - window + 1, read through the block table (this step's own rows were
// written before).  Rows are walked in tiles of 64 from lo with a running maximum and sum, so a position's result
// does not depend on how its sequence was cut into steps.
//
//   s_u = (q~ . row_u) * scale over all D = c + r columns;  o = sum_u softmax(s)_u row_u[:c]
//
// qa (T, H D); out (T, H c); cache (pages, page_size, D).
#define LAT_MAX_C 2048

template <typename T>
__global__ void attention_latent_kernel(const T* __restrict__ qa, const T* __restrict__ cache,
                                        const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                        const int* __restrict__ block_table, int max_blocks, int page_size, int window,
                                        float scale, T* __restrict__ out, int H, int c, int D) {
  extern __shared__ float qs[];      // D floats
  __shared__ float ps[64];
  __shared__ long rowoff[64];
  const int lane = threadIdx.x, t = blockIdx.x, h = blockIdx.y;
  const int pos = positions[t];
  const int* bt = block_table + (size_t)seq_of_token[t] * max_blocks;
  for (int j = lane; j < D; j += 64) qs[j] = to_f32(qa[((size_t)t * H + h) * D + j]);
  __syncthreads();
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[LAT_MAX_C / 64];
#pragma unroll
  for (int i = 0; i < LAT_MAX_C / 64; ++i) acc[i] = 0.f;
  for (int base = lo; base <= pos; base += 64) {
    const int u = base + lane;
    float s = -INFINITY;
    long off = 0;
    if (u <= pos) {
      off = ((long)bt[u / page_size] * page_size + u % page_size) * D;
      const T* kr = cache + off;
      float dot = 0.f;
      for (int j = 0; j < D; ++j) dot += qs[j] * to_f32(kr[j]);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = u <= pos ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    ps[lane] = p;
    rowoff[lane] = off;
    __syncthreads();
    const int nk = pos - base + 1 < 64 ? pos - base + 1 : 64;
#pragma unroll
    for (int i = 0; i < LAT_MAX_C / 64; ++i) {
      const int j = lane + 64 * i;
      if (j < c) {
        float a = acc[i] * alpha;
        for (int k = 0; k < nk; ++k) a += ps[k] * to_f32(cache[rowoff[k] + j]);
        acc[i] = a;
      }
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < LAT_MAX_C / 64; ++i) {
    const int j = lane + 64 * i;
    if (j < c) out[((size_t)t * H + h) * c + j] = from_f32<T>(acc[i] * inv);
  }
}

extern "C" int gs_attention_latent(const void* qa, const void* cache, int dtype, const int* positions,
                                   const int* seq_of_token, const int* block_table, int max_blocks, int page_size,
                                   int window, float scale, void* out, int ntok, int H, int c, int r,
                                   hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && H > 0 && c > 0 && r >= 0, "attention_latent: bad sizes T=%d H=%d c=%d r=%d", ntok, H, c, r);
  GS_REQUIRE(c <= LAT_MAX_C && c + r <= 12288, "attention_latent: latent rows of %d + %d above the kernel's limit", c, r);
  GS_REQUIRE(H <= 65535, "attention_latent: more than 65535 heads");
  GS_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attention_latent: bad page_size/max_blocks/window");
  if (ntok == 0) return 0;
  const int D = c + r;
  dim3 grid(ntok, H);
  if (dtype == GS_F32)
    attention_latent_kernel<float><<<grid, 64, D * sizeof(float), stream>>>(
        (const float*)qa, (const float*)cache, positions, seq_of_token, block_table, max_blocks, page_size, window, scale,
        (float*)out, H, c, D);
  else if (dtype == GS_BF16)
    attention_latent_kernel<bf16><<<grid, 64, D * sizeof(float), stream>>>(
        (const bf16*)qa, (const bf16*)cache, positions, seq_of_token, block_table, max_blocks, page_size, window, scale,
        (bf16*)out, H, c, D);
  else
    GS_REQUIRE(false, "attention_latent: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("attention_latent");
  return 0;
}
