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
// `vec`: parts are whole runs of eight elements and `w` and `o` allow 16-byte accesses; the lanes then take eight
// neighbours at a time (another fixed order of the same sums).
template <typename TO>
__device__ __forceinline__ void scale_part(const float* p, const float* __restrict__ w, TO* __restrict__ o, float inv,
                                           int first, int step, int hg, bool vec) {
  if (vec) {
    for (int j = first * 8; j < hg; j += step * 8) {
      float w8[8], v[8];
      load8f(w + j, w8);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = p[j + e] * inv * w8[e];
      store8f(o + j, v);
    }
  } else {
    for (int j = first; j < hg; j += step) o[j] = from_f32<TO>(p[j] * inv * w[j]);
  }
}

__device__ __forceinline__ float square_sum(const float* p, int first, int step, int hg, bool vec) {
  float ss = 0.f;
  if (vec) {
    for (int j = first * 8; j < hg; j += step * 8) {
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(p[j + e], p[j + e], ss);
    }
  } else {
    for (int j = first; j < hg; j += step) ss = fmaf(p[j], p[j], ss);
  }
  return ss;
}

template <typename TO>
__device__ __forceinline__ void norm_parts(const float* xs, const float* __restrict__ w, float eps, int groups, int H,
                                           TO* __restrict__ o, float* part_sums, bool vec) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int hg = H / groups;
  const int share = nw / groups;              // wavefronts a part
  if (share >= 2) {
    const int g = wave / share, sub = wave % share;
    const bool mine = g < groups;
    const float* p = xs + (size_t)(mine ? g : 0) * hg;
    float ss = mine ? square_sum(p, sub * 64 + lane, 64 * share, hg, vec) : 0.f;
    ss = wave_sum(ss);
    if (lane == 0) part_sums[wave] = ss;
    __syncthreads();
    if (!mine) return;
    float all = 0.f;
    for (int i = 0; i < share; ++i) all += part_sums[g * share + i];
    scale_part<TO>(p, w + (size_t)g * hg, o + (size_t)g * hg, norm_inverse(all, (float)hg, eps), sub * 64 + lane, 64 * share, hg, vec);
    return;
  }
  for (int g = wave; g < groups; g += nw) {
    const float* p = xs + (size_t)g * hg;
    const float ss = wave_sum(square_sum(p, lane, 64, hg, vec));
    scale_part<TO>(p, w + (size_t)g * hg, o + (size_t)g * hg, norm_inverse(ss, (float)hg, eps), lane, 64, hg, vec);
  }
}

template <typename TD, typename TO>
__global__ void add_group_rmsnorm_kernel(float* __restrict__ res, const TD* __restrict__ d1, const TD* __restrict__ d2,
                                         const float* __restrict__ w, float eps, int groups, TO* __restrict__ out,
                                         const int* __restrict__ rows, int H, int vec) {
  extern __shared__ float gn_row[];
  __shared__ float part_sums[4];
  const int r = blockIdx.x;
  const int s = rows ? rows[r] : r;
  float* x = res + (size_t)s * H;
  const TD* a = d1 ? d1 + (size_t)s * H : nullptr;
  const TD* b = d2 ? d2 + (size_t)s * H : nullptr;
  if (vec) {
    for (int j = threadIdx.x * 8; j < H; j += blockDim.x * 8) {
      float v[8], d[8];
      load8f(x + j, v);
      if (a) {
        load8f(a + j, d);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += d[e];
      }
      if (b) {
        load8f(b + j, d);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += d[e];
      }
      if ((a || b) && !rows) store8f(x + j, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) gn_row[j + e] = v[e];
    }
  } else {
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
      float v = x[j];
      if (a) v += to_f32(a[j]);
      if (b) v += to_f32(b[j]);
      if ((a || b) && !rows) x[j] = v;
      gn_row[j] = v;
    }
  }
  __syncthreads();
  norm_parts<TO>(gn_row, w, eps, groups, H, out + (size_t)r * H, part_sums, vec);
}

template <typename TZ, typename TO>
__global__ void gated_group_norm_kernel(const float* __restrict__ y, const TZ* __restrict__ z, int ldz,
                                        const float* __restrict__ w, float eps, int groups, TO* __restrict__ out, int H,
                                        int vec) {
  extern __shared__ float gn_row[];
  __shared__ float part_sums[4];
  const int r = blockIdx.x;
  if (vec) {
    for (int j = threadIdx.x * 8; j < H; j += blockDim.x * 8) {
      float g[8], v[8];
      load8f(z + (size_t)r * ldz + j, g);
      load8f(y + (size_t)r * H + j, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) gn_row[j + e] = v[e] * (g[e] / (1.f + expf(-g[e])));
    }
  } else {
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
      const float g = to_f32(z[(size_t)r * ldz + j]);
      gn_row[j] = y[(size_t)r * H + j] * (g / (1.f + expf(-g)));
    }
  }
  __syncthreads();
  norm_parts<TO>(gn_row, w, eps, groups, H, out + (size_t)r * H, part_sums, vec);
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
  const int vec = (H / groups) % 8 == 0 &&
                  (((uintptr_t)res | (uintptr_t)d1 | (uintptr_t)d2 | (uintptr_t)w | (uintptr_t)out) & 15) == 0;
#define GS_RUN(TD, TO)                                                                                             \
  add_group_rmsnorm_kernel<TD, TO><<<n_out, threads, lds, stream>>>(res, (const TD*)d1, (const TD*)d2, w, eps, groups, \
                                                                    (TO*)out, rows, H, vec)
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
  const int vec = (H / groups) % 8 == 0 && ldz % 8 == 0 &&
                  (((uintptr_t)y | (uintptr_t)z | (uintptr_t)w | (uintptr_t)out) & 15) == 0;
#define GS_RUN(TZ, TO)                                                                                             \
  gated_group_norm_kernel<TZ, TO><<<T, threads, lds, stream>>>(y, (const TZ*)z, ldz, w, eps, groups, (TO*)out, H, vec)
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
