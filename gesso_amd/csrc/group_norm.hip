// RMS norms over equal consecutive parts of a row ("groups"): each part is divided by its own root mean square.
//
//   add_group_rmsnorm   x = res[s] (+ d1[s]) (+ d2[s]), written back unless rows are gathered;
//                       out[r, part g] = x_g / sqrt(mean(x_g^2) + eps) * w_g          one block per output row
//   gated_group_norm    v = y * silu(z) (float32), then the same norm in parts         one block per row
//
// The row is staged in LDS as float32; a wavefront takes a part at a time (or, with fewer parts than wavefronts, a
// share of one): its lanes walk the part together, each lane summing its elements in ascending order, the lanes' and
// wavefronts' sums are added in a fixed order.  So a row's result depends on the row alone.  All arithmetic is float32.
#include "common.h"

// Norm of the parts of a staged row `xs` (H floats in LDS), written to `o`.  Blocks are four wavefronts: with four
// parts or more a wavefront takes a part at a time; with one or two parts, four or two wavefronts share a part (each
// sums every fourth or second run of 64 elements, the wavefronts' sums are added in ascending order).  `part_sums`:
// four floats of LDS.  Every thread of the block must call this.
template <typename TO>
__device__ __forceinline__ void norm_parts(const float* xs, const float* __restrict__ w, float eps, int groups, int H,
                                           TO* __restrict__ o, float* part_sums) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int hg = H / groups;
  const int share = nw / groups;              // wavefronts a part
  if (share >= 2) {
    const int g = wave / share, sub = wave % share;
    const bool mine = g < groups;
    const float* p = xs + (size_t)(mine ? g : 0) * hg;
    float ss = 0.f;
    if (mine)
      for (int j = sub * 64 + lane; j < hg; j += 64 * share) ss = fmaf(p[j], p[j], ss);
    ss = wave_sum(ss);
    if (lane == 0) part_sums[wave] = ss;
    __syncthreads();
    if (!mine) return;
    float all = 0.f;
    for (int i = 0; i < share; ++i) all += part_sums[g * share + i];
    const float inv = norm_inverse(all, (float)hg, eps);
    for (int j = sub * 64 + lane; j < hg; j += 64 * share) o[(size_t)g * hg + j] = from_f32<TO>(p[j] * inv * w[(size_t)g * hg + j]);
    return;
  }
  for (int g = wave; g < groups; g += nw) {
    const float* p = xs + (size_t)g * hg;
    float ss = 0.f;
    for (int j = lane; j < hg; j += 64) ss = fmaf(p[j], p[j], ss);
    ss = wave_sum(ss);
    const float inv = norm_inverse(ss, (float)hg, eps);
    for (int j = lane; j < hg; j += 64) o[(size_t)g * hg + j] = from_f32<TO>(p[j] * inv * w[(size_t)g * hg + j]);
  }
}

template <typename TD, typename TO>
__global__ void add_group_rmsnorm_kernel(float* __restrict__ res, const TD* __restrict__ d1, const TD* __restrict__ d2,
                                         const float* __restrict__ w, float eps, int groups, TO* __restrict__ out,
                                         const int* __restrict__ rows, int H) {
  extern __shared__ float gn_row[];
  __shared__ float part_sums[4];
  const int r = blockIdx.x;
  const int s = rows ? rows[r] : r;
  float* x = res + (size_t)s * H;
  const TD* a = d1 ? d1 + (size_t)s * H : nullptr;
  const TD* b = d2 ? d2 + (size_t)s * H : nullptr;
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    float v = x[j];
    if (a) v += to_f32(a[j]);
    if (b) v += to_f32(b[j]);
    if ((a || b) && !rows) x[j] = v;
    gn_row[j] = v;
  }
  __syncthreads();
  norm_parts<TO>(gn_row, w, eps, groups, H, out + (size_t)r * H, part_sums);
}

template <typename TZ, typename TO>
__global__ void gated_group_norm_kernel(const float* __restrict__ y, const TZ* __restrict__ z, int ldz,
                                        const float* __restrict__ w, float eps, int groups, TO* __restrict__ out, int H) {
  extern __shared__ float gn_row[];
  __shared__ float part_sums[4];
  const int r = blockIdx.x;
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    const float g = to_f32(z[(size_t)r * ldz + j]);
    gn_row[j] = y[(size_t)r * H + j] * (g / (1.f + expf(-g)));
  }
  __syncthreads();
  norm_parts<TO>(gn_row, w, eps, groups, H, out + (size_t)r * H, part_sums);
}

static int group_norm_threads(int groups, int H) {
  (void)groups;
  (void)H;
  return 256;                                 // four wavefronts (norm_parts counts on it)
}

extern "C" int gs_add_group_rmsnorm(float* res, const void* d1, const void* d2, int delta_dtype, const float* w, float eps,
                                    int groups, void* out, int out_dtype, const int* rows, int n_out, int H,
                                    hipStream_t stream) {
  GS_REQUIRE(n_out >= 0 && H > 0 && groups > 0 && H % groups == 0, "add_group_rmsnorm: bad sizes rows=%d H=%d groups=%d", n_out, H, groups);
  GS_REQUIRE(eps > 0.f, "add_group_rmsnorm: eps must be positive");
  GS_REQUIRE((size_t)H * sizeof(float) <= 65536, "add_group_rmsnorm: rows of %d are wider than the kernel stages", H);
  if (n_out == 0) return 0;
  const int threads = group_norm_threads(groups, H);
  const size_t lds = (size_t)H * sizeof(float);
#define GS_RUN(TD, TO)                                                                                             \
  add_group_rmsnorm_kernel<TD, TO><<<n_out, threads, lds, stream>>>(res, (const TD*)d1, (const TD*)d2, w, eps, groups, \
                                                                    (TO*)out, rows, H)
  if (delta_dtype == GS_F32 && out_dtype == GS_F32)
    GS_RUN(float, float);
  else if (delta_dtype == GS_BF16 && out_dtype == GS_BF16)
    GS_RUN(bf16, bf16);
  else if (delta_dtype == GS_F32 && out_dtype == GS_BF16)
    GS_RUN(float, bf16);
  else if (delta_dtype == GS_BF16 && out_dtype == GS_F32)
    GS_RUN(bf16, float);
  else
    GS_REQUIRE(false, "add_group_rmsnorm: unknown dtypes %d %d", delta_dtype, out_dtype);
#undef GS_RUN
  GS_LAUNCH_CHECK("add_group_rmsnorm");
  return 0;
}

extern "C" int gs_gated_group_norm(const float* y, const void* z, int z_dtype, int ldz, const float* w, float eps,
                                   int groups, void* out, int out_dtype, int T, int H, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && H > 0 && groups > 0 && H % groups == 0 && ldz >= H, "gated_group_norm: bad sizes rows=%d H=%d groups=%d ldz=%d", T, H, groups, ldz);
  GS_REQUIRE(eps > 0.f, "gated_group_norm: eps must be positive");
  GS_REQUIRE((size_t)H * sizeof(float) <= 65536, "gated_group_norm: rows of %d are wider than the kernel stages", H);
  if (T == 0) return 0;
  const int threads = group_norm_threads(groups, H);
  const size_t lds = (size_t)H * sizeof(float);
#define GS_RUN(TZ, TO)                                                                                             \
  gated_group_norm_kernel<TZ, TO><<<T, threads, lds, stream>>>(y, (const TZ*)z, ldz, w, eps, groups, (TO*)out, H)
  if (z_dtype == GS_F32 && out_dtype == GS_F32)
    GS_RUN(float, float);
  else if (z_dtype == GS_BF16 && out_dtype == GS_BF16)
    GS_RUN(bf16, bf16);
  else
    GS_REQUIRE(false, "gated_group_norm: unknown dtypes %d %d", z_dtype, out_dtype);
#undef GS_RUN
  GS_LAUNCH_CHECK("gated_group_norm");
  return 0;
}
