// A mixture of gated feed-forwards chosen by a router over the token's own features.
//
//   z = W_r x (float32), s = softmax(z) over all router outputs (or, with score_fn 1, s = sigmoid(z), each output for
//   itself); the `top` outputs with the largest s + correction are chosen; the chosen ones' weights are their s divided
//   by the sum of the chosen s (+ 1e-20), or, without `renorm`, their s as they are; both times route_scale.  Outputs e >= E name no
//   expert with weights: such an "identity expert" gives back its input.  An expert is
//     g = min(W_gate x, limit), u = clamp(W_up x, -limit, limit), y = W_down (g sigmoid(alpha g) (u + 1)).
//   Expert weights lie stacked: gate_up (E, 2F, H) (a gate's rows, then the up rows), down (E, H, F).
//
//   moe_router         one block per token, a wavefront for every four router rows: logits by wavefronts that walk
//                      their rows together (float32 sums in a fixed order), softmax, choice and weights by the first
//   clamped_glu        (rows, 2F) = gate | up  ->  (rows, F), the expert's activation; float32 arithmetic
//   moe_routed_up      a[t, k, :] = activation of expert e_k's gate and up products    one block per (token, choice)
//   moe_routed_down    y[t, :] = sum_k w_k (W_down[e_k] a[t, k, :] or x[t, :]) (+ shared[t, :])
//   moe_routed_combine the same sum over the rows that the grouped products (moe_group.hip) left, by place
//
// Token by token only the chosen experts' weights are read; steps of many tokens sort their (token, choice) pairs by
// expert (moe_route with a table of choices) and read every expert's weights once.
#include "common.h"

__device__ __forceinline__ float clamped_glu(float g, float u, float limit, float alpha) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + 1.f);
}

// A row of H values into LDS as float32, by the whole block: 16-byte reads where the row allows them.
template <typename T>
__device__ __forceinline__ void stage_row(float* xs, const T* __restrict__ row, int H) {
  if ((H & 7) == 0 && aligned16(row)) {
    for (int j = threadIdx.x * 8; j < H; j += blockDim.x * 8) {
      float v[8];
      load8f(row + j, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) xs[j + e] = v[e];
    }
  } else {
    for (int j = threadIdx.x; j < H; j += blockDim.x) xs[j] = to_f32(row[j]);
  }
}

// One wavefront, from a token's logits in `z` (LDS, EA floats; `cs` as many, `chosen` top ints): the scores (softmax
// over the outputs, or each output's sigmoid), the `top` largest corrected scores (of equal ones the lowest index), the
// chosen ones' weights.
__device__ __forceinline__ void route_from_logits(float* z, float* cs, int* chosen, const float* __restrict__ correction,
                                                  int top, int EA, int lane, int t, int* __restrict__ choice,
                                                  float* __restrict__ weight, int score_fn, int renorm,
                                                  float route_scale) {
  if (score_fn == 1) {
    for (int e = lane; e < EA; e += 64) {
      z[e] = 1.f / (1.f + expf(-z[e]));
      cs[e] = z[e] + (correction ? correction[e] : 0.f);
    }
  } else {
    float m = -INFINITY;
    for (int e = lane; e < EA; e += 64) m = fmaxf(m, z[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < EA; e += 64) {
      const float p = expf(z[e] - m);
      z[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < EA; e += 64) {
      z[e] = z[e] / sum;
      cs[e] = z[e] + (correction ? correction[e] : 0.f);
    }
  }
  // the largest choice score `top` times over; of equal scores the lowest index
  float picked = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = EA;
    for (int e = lane; e < EA; e += 64) {
      const float v = cs[e];
      if (v > best) {
        best = v;
        at = e;
      }
    }
    const float all = wave_max(best);
    int cand = best == all ? at : EA;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const int other = __shfl_xor(cand, o, GS_WAVE);
      cand = other < cand ? other : cand;
    }
    if (cand >= EA) cand = 0;                 // a row of NaN: any expert, the weights stay NaN
    // (every lane holds the same choice and writes it: each then reads back what it has itself stored)
    cs[cand] = -INFINITY;
    chosen[k] = cand;
    picked += z[cand];
  }
  const float inv = (renorm ? 1.f / (picked + 1e-20f) : 1.f) * route_scale;
  for (int k = lane; k < top; k += 64) {
    choice[(size_t)t * top + k] = chosen[k];
    weight[(size_t)t * top + k] = z[chosen[k]] * inv;
  }
}

template <typename T, typename TW>
__global__ __launch_bounds__(1024) void moe_router_kernel(const T* __restrict__ x, int ldx, const TW* __restrict__ wr,
                                                         const float* __restrict__ correction, int top, int EA, int H,
                                                         int* __restrict__ choice, float* __restrict__ weight,
                                                         int score_fn, int renorm, float route_scale) {
  extern __shared__ float mr_sh[];           // H floats of the row, EA logits, EA choice scores, top chosen outputs
  float* xs = mr_sh;
  float* z = mr_sh + H;
  float* cs = z + EA;
  int* chosen = reinterpret_cast<int*>(cs + EA);
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  stage_row(xs, x + (size_t)t * ldx, H);
  __syncthreads();
  const bool vec = (H & 7) == 0 && aligned16(wr);
  // four rows of the router at a time per wavefront: their loads are in flight together, the token's features are read
  // from LDS once for the four.  Each row's sum runs in the order it would run alone.
  for (int e0 = wave * 4; e0 < EA; e0 += nw * 4) {
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    const TW* row[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) row[r] = wr + (size_t)(e0 + r < EA ? e0 + r : e0) * H;
    if (vec) {
      // two steps of 512 columns at a time: eight loads in flight a lane
      for (int j = lane * 8; j < H; j += 1024) {
        const bool two = j + 512 < H;
        float w8[2][4][8];
#pragma unroll
        for (int r = 0; r < 4; ++r) load8f(row[r] + j, w8[0][r]);
#pragma unroll
        for (int r = 0; r < 4; ++r) load8f(row[r] + (two ? j + 512 : j), w8[1][r]);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          if (u == 1 && !two) break;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float xv = xs[j + 512 * u + i];
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] = fmaf(w8[u][r][i], xv, s[r]);
          }
        }
      }
    } else {
      for (int j = lane; j < H; j += 64) {
        const float xv = xs[j];
#pragma unroll
        for (int r = 0; r < 4; ++r) s[r] = fmaf(to_f32(row[r][j]), xv, s[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float all = wave_sum(s[r]);
      if (lane == 0 && e0 + r < EA) z[e0 + r] = all;
    }
  }
  __syncthreads();
  if (wave != 0) return;
  route_from_logits(z, cs, chosen, correction, top, EA, lane, t, choice, weight, score_fn, renorm, route_scale);
}

template <typename TI, typename TO>
__global__ void clamped_glu_kernel(const TI* __restrict__ in, TO* __restrict__ out, int F, long total, float limit,
                                   float alpha) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long r = i / F;
  const int f = (int)(i % F);
  out[i] = from_f32<TO>(clamped_glu(to_f32(in[r * 2 * F + f]), to_f32(in[r * 2 * F + F + f]), limit, alpha));
}

template <typename T, typename TW>
__global__ void moe_routed_up_kernel(const T* __restrict__ x, int ldx, const int* __restrict__ choice, int top, int E,
                                     const TW* __restrict__ gate_up, int F, int H, float limit, float alpha,
                                     T* __restrict__ a) {
  extern __shared__ float xs[];      // H floats
  const int t = blockIdx.x / top, k = blockIdx.x % top;
  const int e = choice[(size_t)t * top + k];
  if (e >= E) return;                // an identity expert has no inner values
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  stage_row(xs, x + (size_t)t * ldx, H);
  __syncthreads();
  const TW* w = gate_up + (size_t)e * 2 * F * H;
  T* dst = a + ((size_t)t * top + k) * F;
  const bool vec = (H & 7) == 0 && aligned16(w);
  for (int f = blockIdx.y * nw + wave; f < F; f += gridDim.y * nw) {
    const TW* rg = w + (size_t)f * H;
    const TW* ru = w + (size_t)(F + f) * H;
    float sg = 0.f, su = 0.f;
    if (vec) {
      for (int j = lane * 8; j < H; j += 512) {
        float g8[8], u8[8];
        load8f(rg + j, g8);
        load8f(ru + j, u8);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          sg = fmaf(g8[i], xs[j + i], sg);
          su = fmaf(u8[i], xs[j + i], su);
        }
      }
    } else {
      for (int j = lane; j < H; j += 64) {
        sg = fmaf(to_f32(rg[j]), xs[j], sg);
        su = fmaf(to_f32(ru[j]), xs[j], su);
      }
    }
    sg = wave_sum(sg);
    su = wave_sum(su);
    // the products are stored in the activation type before the activation, as products of their own would be
    if (lane == 0) dst[f] = from_f32<T>(clamped_glu(to_f32(from_f32<T>(sg)), to_f32(from_f32<T>(su)), limit, alpha));
  }
}

template <typename T, typename TW>
__global__ void moe_routed_down_kernel(const T* __restrict__ a, const T* __restrict__ x, int ldx,
                                       const int* __restrict__ choice, const float* __restrict__ weight, int top, int E,
                                       const TW* __restrict__ down, int F, int H, const T* __restrict__ shared,
                                       T* __restrict__ y) {
  extern __shared__ float as[];      // top * F floats
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int j = threadIdx.x; j < top * F; j += blockDim.x) {
    const bool real = choice[(size_t)t * top + j / F] < E;
    as[j] = real ? to_f32(a[(size_t)t * top * F + j]) : 0.f;
  }
  __syncthreads();
  const bool vec = (F & 7) == 0 && aligned16(down);
  for (int i = blockIdx.y * nw + wave; i < H; i += gridDim.y * nw) {
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = choice[(size_t)t * top + k];
      const float wk = weight[(size_t)t * top + k];
      if (e >= E) {
        total += wk * to_f32(x[(size_t)t * ldx + i]);
        continue;
      }
      const TW* row = down + ((size_t)e * H + i) * F;
      float s = 0.f;
      if (vec) {
        for (int j = lane * 8; j < F; j += 512) {
          float w8[8];
          load8f(row + j, w8);
#pragma unroll
          for (int u = 0; u < 8; ++u) s = fmaf(w8[u], as[k * F + j + u], s);
        }
      } else {
        for (int j = lane; j < F; j += 64) s = fmaf(to_f32(row[j]), as[k * F + j], s);
      }
      total += wk * wave_sum(s);
    }
    if (lane == 0) {
      if (shared) total += to_f32(shared[(size_t)t * H + i]);
      y[(size_t)t * H + i] = from_f32<T>(total);
    }
  }
}

template <typename T>
__global__ void moe_routed_combine_kernel(const float* __restrict__ ys, const int* __restrict__ place_of,
                                          const float* __restrict__ weight, int top, const T* __restrict__ x, int ldx,
                                          const T* __restrict__ shared, T* __restrict__ y, int H) {
  const int t = blockIdx.x;
  if ((H & 7) == 0 && (ldx & 7) == 0 && aligned16(ys) && aligned16(x) && aligned16(y) && (!shared || aligned16(shared))) {
    // eight columns a thread, 16-byte accesses; every column's sum in the order of the loop below
    for (int j = threadIdx.x * 8; j < H; j += blockDim.x * 8) {
      float total[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, v[8];
      for (int k = 0; k < top; ++k) {
        const int place = place_of[(size_t)t * top + k];
        if (place >= 0) load8f(ys + (size_t)place * H + j, v);
        else load8f(x + (size_t)t * ldx + j, v);
        const float wk = weight[(size_t)t * top + k];
#pragma unroll
        for (int e = 0; e < 8; ++e) total[e] += wk * v[e];
      }
      if (shared) {
        load8f(shared + (size_t)t * H + j, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) total[e] += v[e];
      }
      store8f(y + (size_t)t * H + j, total);
    }
    return;
  }
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
      const int place = place_of[(size_t)t * top + k];
      const float v = place >= 0 ? ys[(size_t)place * H + j] : to_f32(x[(size_t)t * ldx + j]);
      total += weight[(size_t)t * top + k] * v;
    }
    if (shared) total += to_f32(shared[(size_t)t * H + j]);
    y[(size_t)t * H + j] = from_f32<T>(total);
  }
}

static int moe_routed_blocks_y(int outputs, int tokens) {
  // enough blocks to fill the chip when tokens are few, one block a token when they are many
  int y = gs_ceil_div(outputs, 4);
  int cap = 2048 / (tokens > 0 ? tokens : 1);
  if (cap < 1) cap = 1;
  return y < cap ? y : cap;
}

extern "C" int gs_moe_router(const void* x, int dtype, int ldx, const void* wr, int w_dtype, const float* correction,
                             int top, int EA, int H, int* choice, float* weight, int ntok, int score_fn, int renorm,
                             float route_scale, hipStream_t stream) {
  GS_REQUIRE(score_fn == 0 || score_fn == 1, "moe_router: scores are a softmax (0) or sigmoids (1), not %d", score_fn);
  GS_REQUIRE(ntok >= 0 && top > 0 && EA >= top && H > 0 && ldx >= H, "moe_router: bad sizes T=%d top=%d outputs=%d H=%d", ntok, top, EA, H);
  const size_t lds = ((size_t)H + 2 * (size_t)EA + (size_t)top) * sizeof(float);
  GS_REQUIRE(lds <= 65536, "moe_router: rows of %d and %d outputs are more than the kernel stages", H, EA);
  if (ntok == 0) return 0;
  // a wavefront for every four router rows, so that one pass over the token's features serves them all (up to 16)
  const int threads = 64 * (gs_ceil_div(EA, 4) < 16 ? (gs_ceil_div(EA, 4) < 4 ? 4 : gs_ceil_div(EA, 4)) : 16);
  if (dtype == GS_F32 && w_dtype == GS_F32)
    moe_router_kernel<float, float><<<ntok, threads, lds, stream>>>((const float*)x, ldx, (const float*)wr, correction, top,
                                                                EA, H, choice, weight, score_fn, renorm, route_scale);
  else if (dtype == GS_BF16 && w_dtype == GS_BF16)
    moe_router_kernel<bf16, bf16><<<ntok, threads, lds, stream>>>((const bf16*)x, ldx, (const bf16*)wr, correction, top, EA, H,
                                                              choice, weight, score_fn, renorm, route_scale);
  else if (dtype == GS_BF16 && w_dtype == GS_F32)
    moe_router_kernel<bf16, float><<<ntok, threads, lds, stream>>>((const bf16*)x, ldx, (const float*)wr, correction, top, EA,
                                                               H, choice, weight, score_fn, renorm, route_scale);
  else
    GS_REQUIRE(false, "moe_router: unsupported types %d %d", dtype, w_dtype);
  GS_LAUNCH_CHECK("moe_router");
  return 0;
}

extern "C" int gs_clamped_glu(const void* in, int in_dtype, void* out, int out_dtype, long rows, int F, float limit,
                              float alpha, hipStream_t stream) {
  GS_REQUIRE(rows >= 0 && F > 0, "clamped_glu: bad sizes rows=%ld F=%d", rows, F);
  if (rows == 0) return 0;
  const long total = rows * F;
  const int blocks = gs_ceil_div(total, 256);
  if (in_dtype == GS_F32 && out_dtype == GS_F32)
    clamped_glu_kernel<float, float><<<blocks, 256, 0, stream>>>((const float*)in, (float*)out, F, total, limit, alpha);
  else if (in_dtype == GS_BF16 && out_dtype == GS_BF16)
    clamped_glu_kernel<bf16, bf16><<<blocks, 256, 0, stream>>>((const bf16*)in, (bf16*)out, F, total, limit, alpha);
  else if (in_dtype == GS_F32 && out_dtype == GS_BF16)
    clamped_glu_kernel<float, bf16><<<blocks, 256, 0, stream>>>((const float*)in, (bf16*)out, F, total, limit, alpha);
  else
    GS_REQUIRE(false, "clamped_glu: unsupported types %d %d", in_dtype, out_dtype);
  GS_LAUNCH_CHECK("clamped_glu");
  return 0;
}

extern "C" int gs_moe_routed_up(const void* x, int dtype, int ldx, const int* choice, int top, int E, const void* gate_up,
                                int w_dtype, int F, int H, float limit, float alpha, void* a, int ntok,
                                hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && top > 0 && F > 0 && H > 0 && ldx >= H && E >= 0, "moe_routed_up: bad sizes T=%d top=%d F=%d H=%d", ntok, top, F, H);
  GS_REQUIRE(H * sizeof(float) <= 65536, "moe_routed_up: rows of %d are wider than the kernel's staging", H);
  if (ntok == 0 || E == 0) return 0;
  dim3 grid(ntok * top, moe_routed_blocks_y(F, ntok * top));
  const size_t lds = H * sizeof(float);
#define GS_RUN(T, TW)                                                                                                 \
  moe_routed_up_kernel<T, TW><<<grid, 256, lds, stream>>>((const T*)x, ldx, choice, top, E, (const TW*)gate_up, F, H, \
                                                          limit, alpha, (T*)a)
  if (dtype == GS_F32 && w_dtype == GS_F32)
    GS_RUN(float, float);
  else if (dtype == GS_BF16 && w_dtype == GS_BF16)
    GS_RUN(bf16, bf16);
  else if (dtype == GS_BF16 && w_dtype == GS_F32)
    GS_RUN(bf16, float);
  else
    GS_REQUIRE(false, "moe_routed_up: unsupported types %d %d", dtype, w_dtype);
#undef GS_RUN
  GS_LAUNCH_CHECK("moe_routed_up");
  return 0;
}

extern "C" int gs_moe_routed_down(const void* a, int dtype, const void* x, int ldx, const int* choice,
                                  const float* weight, int top, int E, const void* down, int w_dtype, int F, int H,
                                  const void* shared, void* y, int ntok, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && top > 0 && F > 0 && H > 0 && ldx >= H, "moe_routed_down: bad sizes T=%d top=%d F=%d H=%d", ntok, top, F, H);
  GS_REQUIRE((long)top * F * sizeof(float) <= 65536, "moe_routed_down: %d x %d inner values are more than the kernel stages", top, F);
  if (ntok == 0) return 0;
  dim3 grid(ntok, moe_routed_blocks_y(H, ntok));
  const size_t lds = (size_t)top * F * sizeof(float);
#define GS_RUN(T, TW)                                                                                                   \
  moe_routed_down_kernel<T, TW><<<grid, 256, lds, stream>>>((const T*)a, (const T*)x, ldx, choice, weight, top, E,      \
                                                            (const TW*)down, F, H, (const T*)shared, (T*)y)
  if (dtype == GS_F32 && w_dtype == GS_F32)
    GS_RUN(float, float);
  else if (dtype == GS_BF16 && w_dtype == GS_BF16)
    GS_RUN(bf16, bf16);
  else if (dtype == GS_BF16 && w_dtype == GS_F32)
    GS_RUN(bf16, float);
  else
    GS_REQUIRE(false, "moe_routed_down: unsupported types %d %d", dtype, w_dtype);
#undef GS_RUN
  GS_LAUNCH_CHECK("moe_routed_down");
  return 0;
}

extern "C" int gs_moe_routed_combine(const float* ys, const int* place_of, const float* weight, int top, const void* x,
                                     int ldx, const void* shared, void* y, int dtype, int T, int H, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && top > 0 && H > 0 && ldx >= H, "moe_routed_combine: bad sizes T=%d top=%d H=%d", T, top, H);
  if (T == 0) return 0;
  if (dtype == GS_BF16)
    moe_routed_combine_kernel<bf16><<<T, 256, 0, stream>>>(ys, place_of, weight, top, (const bf16*)x, ldx,
                                                           (const bf16*)shared, (bf16*)y, H);
  else if (dtype == GS_F32)
    moe_routed_combine_kernel<float><<<T, 256, 0, stream>>>(ys, place_of, weight, top, (const float*)x, ldx,
                                                            (const float*)shared, (float*)y, H);
  else
    GS_REQUIRE(false, "moe_routed_combine: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("moe_routed_combine");
  return 0;
}
