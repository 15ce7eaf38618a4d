// Layer norm of the residual stream, the sum of two normed branches, and a gate on rows of heads.
//
// add_layernorm: one block per output row r; source row s = rows ? rows[r] : r.
//   x = res[s] (+ delta[s]);  out[r] = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w + b
//   Without `rows` the sum is written back to res (the stream moves on); with `rows` (a gather at the model's end) res
//   is left as it is.  The row is staged in LDS as float32: the mean first, then the mean of the squared deviations from
//   it (not the difference of two large sums).
// normed_pair_sum: out = sa * rms(a) * wa + sb * rms(b) * wb, a and b float32 rows of two branches' last products,
//   rms(x) = x / sqrt(mean(x^2) + eps); one rounding, at the end.
// gated_rows: out = o * g(gate), g = sigmoid (0) or silu (1); the gate stands in rows (T, ldg) from column og on.
#include "common.h"

template <typename TD, typename TO>
__global__ void add_layernorm_kernel(float* __restrict__ res, const TD* __restrict__ delta, const float* __restrict__ w,
                                     const float* __restrict__ b, float eps, TO* __restrict__ out,
                                     const int* __restrict__ rows, int H) {
  extern __shared__ float ln_row[];
  __shared__ float red[17];
  const int r = blockIdx.x;
  const int s = rows ? rows[r] : r;
  float* x = res + (size_t)s * H;
  const TD* dl = delta ? delta + (size_t)s * H : nullptr;
  float sum = 0.f;
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    float v = x[j];
    if (dl) {
      v += to_f32(dl[j]);
      if (!rows) x[j] = v;
    }
    ln_row[j] = v;
    sum += v;
  }
  const float mean = block_sum(sum, red) / (float)H;
  float ss = 0.f;
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    const float dv = ln_row[j] - mean;
    ss += dv * dv;
  }
  ss = block_sum(ss, red);
  const float inv = norm_inverse(ss, (float)H, eps);
  TO* o = out + (size_t)r * H;
  for (int j = threadIdx.x; j < H; j += blockDim.x)
    o[j] = from_f32<TO>((ln_row[j] - mean) * inv * w[j] + (b ? b[j] : 0.f));
}

extern "C" int gs_add_layernorm(float* res, const void* delta, int delta_dtype, const float* w, const float* b, float eps,
                                void* out, int out_dtype, const int* rows, int n_out, int H, hipStream_t stream) {
  GS_REQUIRE(n_out >= 0 && H > 0 && H <= 15360, "add_layernorm: bad sizes rows=%d H=%d (rows of up to 15360 values)", n_out, H);
  GS_REQUIRE(eps > 0.f, "add_layernorm: eps must be positive");
  if (n_out == 0) return 0;
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  const size_t lds = (size_t)H * sizeof(float);
#define GS_RUN(TD, TO) \
  add_layernorm_kernel<TD, TO><<<n_out, threads, lds, stream>>>(res, (const TD*)delta, w, b, eps, (TO*)out, rows, H)
  if (delta_dtype == GS_F32 && out_dtype == GS_F32)
    GS_RUN(float, float);
  else if (delta_dtype == GS_BF16 && out_dtype == GS_BF16)
    GS_RUN(bf16, bf16);
  else if (delta_dtype == GS_F32 && out_dtype == GS_BF16)
    GS_RUN(float, bf16);
  else if (delta_dtype == GS_BF16 && out_dtype == GS_F32)
    GS_RUN(bf16, float);
  else
    GS_REQUIRE(false, "add_layernorm: unknown dtypes %d %d", delta_dtype, out_dtype);
#undef GS_RUN
  GS_LAUNCH_CHECK("add_layernorm");
  return 0;
}

template <typename TO>
__global__ void normed_pair_sum_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                       const float* __restrict__ wa, const float* __restrict__ wb, float eps, float sa,
                                       float sb, TO* __restrict__ out, int W) {
  __shared__ float red[17];
  const float* ra = a + (size_t)blockIdx.x * W;
  const float* rb = b + (size_t)blockIdx.x * W;
  float ssa = 0.f, ssb = 0.f;
  for (int j = threadIdx.x; j < W; j += blockDim.x) {
    ssa += ra[j] * ra[j];
    ssb += rb[j] * rb[j];
  }
  ssa = block_sum(ssa, red);
  ssb = block_sum(ssb, red);
  const float ia = sa * norm_inverse(ssa, (float)W, eps), ib = sb * norm_inverse(ssb, (float)W, eps);
  TO* o = out + (size_t)blockIdx.x * W;
  for (int j = threadIdx.x; j < W; j += blockDim.x) o[j] = from_f32<TO>(ra[j] * ia * wa[j] + rb[j] * ib * wb[j]);
}

extern "C" int gs_normed_pair_sum(const float* a, const float* b, const float* wa, const float* wb, float eps, float sa,
                                  float sb, void* out, int out_dtype, int T, int W, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && W > 0, "normed_pair_sum: bad sizes T=%d W=%d", T, W);
  GS_REQUIRE(eps > 0.f, "normed_pair_sum: eps must be positive");
  if (T == 0) return 0;
  const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
  if (out_dtype == GS_F32)
    normed_pair_sum_kernel<float><<<T, threads, 0, stream>>>(a, b, wa, wb, eps, sa, sb, (float*)out, W);
  else if (out_dtype == GS_BF16)
    normed_pair_sum_kernel<bf16><<<T, threads, 0, stream>>>(a, b, wa, wb, eps, sa, sb, (bf16*)out, W);
  else
    GS_REQUIRE(false, "normed_pair_sum: unknown dtype %d", out_dtype);
  GS_LAUNCH_CHECK("normed_pair_sum");
  return 0;
}

template <typename T>
__global__ void gated_rows_kernel(const T* __restrict__ o, const T* __restrict__ gate, int ldg, int og, int act,
                                  T* __restrict__ out, int W, long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long t = i / W;
  const int c = (int)(i - t * W);
  const float z = to_f32(gate[t * ldg + og + c]);
  const float sg = 1.0f / (1.0f + expf(-z));
  out[i] = from_f32<T>(to_f32(o[i]) * (act ? z * sg : sg));
}

extern "C" int gs_gated_rows(const void* o, const void* gate, int dtype, int ldg, int og, int act, void* out, int T,
                             int W, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && W > 0 && og >= 0 && og + W <= ldg, "gated_rows: the gate lies outside the rows of %d", ldg);
  GS_REQUIRE(act == 0 || act == 1, "gated_rows: unknown gate function %d", act);
  if (T == 0) return 0;
  const long total = (long)T * W;
  if (dtype == GS_F32)
    gated_rows_kernel<float><<<gs_ceil_div(total, 256), 256, 0, stream>>>((const float*)o, (const float*)gate, ldg, og,
                                                                           act, (float*)out, W, total);
  else if (dtype == GS_BF16)
    gated_rows_kernel<bf16><<<gs_ceil_div(total, 256), 256, 0, stream>>>((const bf16*)o, (const bf16*)gate, ldg, og, act,
                                                                          (bf16*)out, W, total);
  else
    GS_REQUIRE(false, "gated_rows: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("gated_rows");
  return 0;
}
