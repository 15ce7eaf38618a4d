// Table-routed experts for steps of many tokens: the (token, choice) pairs are sorted by expert on the device, and each
// expert's weights are read once for all of its pairs by a product on the matrix cores.
//
//   moe_route      one block: counts the pairs of every expert, gives each pair its place among its expert's (perm:
//                  place -> token, place_of: pair -> place), and lists the tiles of up to 128 places of one expert
//                  (expert, first place, count) with their number.  Nothing comes back to the host: the products
//                  are launched with as many blocks as tiles can be at most, and blocks past the number return.
//   moe_group_gemm Y[place, :] = W[expert] X[row of place, :] per tile, v_mfma_f32_32x32x16_bf16, 128 x 128 tiles of
//                  four wavefronts, k in steps of 64 through two LDS buffers (the scheme of the product for many rows);
//                  rows are gathered through perm (up-projection, epilogue relu^2 on the rounded product, bfloat16
//                  out) or taken in place order (down-projection, float32 out)
//   moe_combine    y[t, :] = (1 / top) sum_k Y[place_of[t, k], :] (+ sigmoid(g_t) * shared[t, :]), the choices
//                  added in their order, float32, one rounding
//
// A pair's result depends on its own row and its expert's weights alone, whichever rows share its tile.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 mg_bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float mg_f32x16_t;

constexpr int MG_BM = 128, MG_BN = 128, MG_BK = 64, MG_LDR = MG_BK + 8;

__global__ __launch_bounds__(1024) void moe_route_kernel(const int* __restrict__ ids, const int* __restrict__ table,
                                                         int T, int top, int E, int* __restrict__ perm,
                                                         int* __restrict__ place_of, int* __restrict__ tiles,
                                                         int max_tiles, int* __restrict__ n_tiles) {
  extern __shared__ int mg_sh[];          // counts[E], starts[E]
  int* counts = mg_sh;
  int* starts = mg_sh + E;
  const int P = T * top;
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  // (without ids the table holds the choices of the step's own rows; an entry that names no expert takes no place)
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = ids ? table[(size_t)ids[p / top] * top + p % top] : table[p];
    if (e < E) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      const int n = counts[e];
      starts[e] = at;
      for (int r = 0; r < n; r += MG_BM) {
        if (nt < max_tiles) {
          tiles[nt] = e;
          tiles[max_tiles + nt] = at + r;
          tiles[2 * max_tiles + nt] = n - r < MG_BM ? n - r : MG_BM;
        }
        ++nt;
      }
      at += n;
      counts[e] = 0;
    }
    *n_tiles = nt < max_tiles ? nt : max_tiles;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = ids ? table[(size_t)ids[p / top] * top + p % top] : table[p];
    if (e >= E) {
      place_of[p] = -1;
      continue;
    }
    const int place = starts[e] + atomicAdd(&counts[e], 1);
    perm[place] = p / top;
    place_of[p] = place;
  }
}

// EPI 0: float32 out.  EPI 1: bfloat16 out.  EPI 2: relu(bfloat16(v))^2, bfloat16 out.
template <int EPI, typename TOut>
__global__ __launch_bounds__(256) void moe_group_gemm_kernel(const bf16* __restrict__ X, int ldx,
                                                             const int* __restrict__ gather,
                                                             const bf16* __restrict__ W, TOut* __restrict__ Y, int ldy,
                                                             const int* __restrict__ tiles, int max_tiles,
                                                             const int* __restrict__ n_tiles, int N, int K) {
  constexpr int NT = 256, WN = 2;
  constexpr int RM = MG_BM / 2, RN = MG_BN / 2, TM = RM / 32, TN = RN / 32;
  constexpr int LA = MG_BM * 8 / NT, LB = MG_BN * 8 / NT;
  constexpr int STAGE = (MG_BM + MG_BN) * MG_LDR;
  extern __shared__ __align__(16) uint16_t mg_lds[];
  const int t = blockIdx.x;
  if (t >= *n_tiles) return;
  const int expert = tiles[t], row0 = tiles[max_tiles + t], cnt = tiles[2 * max_tiles + t];
  const int n0 = blockIdx.y * MG_BN;
  W += (size_t)expert * N * K;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN, l32 = lane & 31, kh = lane >> 5;
  const int r0 = tid >> 3, c = tid & 7;
  const bf16* ap[LA];
  const bf16* bp[LB];
#pragma unroll
  for (int i = 0; i < LA; ++i) {
    int rr = r0 + i * (NT / 8);
    if (rr >= cnt) rr = cnt - 1;
    const int place = row0 + rr;
    ap[i] = X + (size_t)(gather ? gather[place] : place) * ldx + c * 8;
  }
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    int n = n0 + r0 + i * (NT / 8);
    if (n >= N) n = N - 1;
    bp[i] = W + (size_t)n * K + c * 8;
  }
  uint4 sa[LA], sb[LB];
#define MG_GLOAD_MASKED(k0)                                                                                  \
  {                                                                                                          \
    const bool in = (k0) + c * 8 < K;                                                                        \
    const int kk = in ? (k0) : -c * 8;                                                                       \
    _Pragma("unroll") for (int i = 0; i < LA; ++i) {                                                         \
      sa[i] = *reinterpret_cast<const uint4*>(ap[i] + kk);                                                   \
      sa[i] = in ? sa[i] : make_uint4(0, 0, 0, 0);                                                           \
    }                                                                                                        \
    _Pragma("unroll") for (int i = 0; i < LB; ++i) {                                                         \
      sb[i] = *reinterpret_cast<const uint4*>(bp[i] + kk);                                                   \
      sb[i] = in ? sb[i] : make_uint4(0, 0, 0, 0);                                                           \
    }                                                                                                        \
  }
#define MG_LSTORE(buf)                                                                                       \
  {                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < LA; ++i)                                                           \
        *reinterpret_cast<uint4*>(mg_lds + (buf) * STAGE + (r0 + i * (NT / 8)) * MG_LDR + c * 8) = sa[i];      \
    _Pragma("unroll") for (int i = 0; i < LB; ++i)                                                           \
        *reinterpret_cast<uint4*>(mg_lds + (buf) * STAGE + (MG_BM + r0 + i * (NT / 8)) * MG_LDR + c * 8) = sb[i]; \
  }
#define MG_COMPUTE(buf)                                                                                      \
  {                                                                                                          \
    const uint16_t* a_base = mg_lds + (buf) * STAGE + (wm * RM + l32) * MG_LDR + kh * 8;                     \
    const uint16_t* b_base = mg_lds + (buf) * STAGE + (MG_BM + wn * RN + l32) * MG_LDR + kh * 8;             \
    _Pragma("unroll") for (int ks = 0; ks < MG_BK / 16; ++ks) {                                              \
      mg_bf16x8_t af[TM], bf[TN];                                                                            \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                         \
          af[i] = *reinterpret_cast<const mg_bf16x8_t*>(a_base + i * 32 * MG_LDR + ks * 16);                 \
      _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                         \
          bf[j] = *reinterpret_cast<const mg_bf16x8_t*>(b_base + j * 32 * MG_LDR + ks * 16);                 \
      _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                         \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                       \
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);             \
    }                                                                                                        \
  }
  mg_f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  const int nk = (K + MG_BK - 1) / MG_BK;
  MG_GLOAD_MASKED(0);
  MG_LSTORE(0);
  __syncthreads();
  for (int it = 0; it + 1 < nk; ++it) {
    const int buf = it & 1;
    MG_GLOAD_MASKED((it + 1) * MG_BK);
    MG_COMPUTE(buf);
    MG_LSTORE(buf ^ 1);
    __syncthreads();
  }
  MG_COMPUTE((nk - 1) & 1);
#undef MG_GLOAD_MASKED
#undef MG_LSTORE
#undef MG_COMPUTE
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * RN + j * 32 + l32;
      if (n >= N) continue;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int rr = wm * RM + i * 32 + 8 * (e >> 2) + 4 * kh + (e & 3);
        if (rr >= cnt) continue;
        float v = acc[i][j][e];
        if (EPI == 2) {
          v = to_f32(f32_to_bf16(v));
          v = v > 0.f ? v * v : 0.f;
        }
        Y[(size_t)(row0 + rr) * ldy + n] = from_f32<TOut>(v);
      }
    }
}

template <typename T>
__global__ void moe_combine_kernel(const float* __restrict__ ys, const int* __restrict__ place_of, int top,
                                   const T* __restrict__ shared, const T* __restrict__ gate, int ldg,
                                   T* __restrict__ y, int H) {
  const int t = blockIdx.x;
  const float share = 1.0f / (float)top;
  float g = 0.f;
  if (shared) g = 1.f / (1.f + expf(-to_f32(gate[(size_t)t * ldg])));
  if ((H & 3) == 0) {
    // four columns a thread: 16-byte loads of the experts' rows
    for (int j = threadIdx.x * 4; j < H; j += blockDim.x * 4) {
      float4 total = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int k = 0; k < top; ++k) {
        const float4 v = *reinterpret_cast<const float4*>(ys + (size_t)place_of[(size_t)t * top + k] * H + j);
        total.x += v.x * share; total.y += v.y * share; total.z += v.z * share; total.w += v.w * share;
      }
      float o[4] = {total.x, total.y, total.z, total.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (shared) o[i] += g * to_f32(shared[(size_t)t * H + j + i]);
        y[(size_t)t * H + j + i] = from_f32<T>(o[i]);
      }
    }
    return;
  }
  for (int j = threadIdx.x; j < H; j += blockDim.x) {
    float total = 0.f;
    for (int k = 0; k < top; ++k) total += ys[(size_t)place_of[(size_t)t * top + k] * H + j] * share;
    if (shared) total += g * to_f32(shared[(size_t)t * H + j]);
    y[(size_t)t * H + j] = from_f32<T>(total);
  }
}

extern "C" int gs_moe_group_rows() { return MG_BM; }

extern "C" int gs_moe_route(const int* ids, const int* table, int T, int top, int E, int* perm, int* place_of,
                            int* tiles, int max_tiles, int* n_tiles, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && top > 0 && E > 0 && E <= 4096, "moe_route: bad sizes T=%d top=%d E=%d", T, top, E);
  GS_REQUIRE((long)T * top < (1L << 30), "moe_route: too many pairs");
  GS_REQUIRE(max_tiles >= gs_ceil_div((long)T * top, MG_BM) + E, "moe_route: room for %d tiles is too little", max_tiles);
  if (T == 0) return 0;
  moe_route_kernel<<<1, 1024, 2 * E * sizeof(int), stream>>>(ids, table, T, top, E, perm, place_of, tiles, max_tiles, n_tiles);
  GS_LAUNCH_CHECK("moe_route");
  return 0;
}

extern "C" int gs_moe_group_gemm(const void* X, int ldx, const int* gather, const void* W, void* Y, int y_dtype,
                                 int ldy, const int* tiles, int max_tiles, const int* n_tiles, int N, int K,
                                 int epilogue, hipStream_t stream) {
  GS_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && max_tiles > 0 && max_tiles <= (1 << 30), "moe_group_gemm: bad sizes N=%d K=%d (K a multiple of 8)", N, K);
  GS_REQUIRE(ldx >= K && ldx % 8 == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0 && ldy >= N,
             "moe_group_gemm: X and W 16-byte aligned, row strides %d, %d", ldx, ldy);
  GS_REQUIRE((epilogue == 0 && y_dtype == GS_F32) || ((epilogue == 1 || epilogue == 2) && y_dtype == GS_BF16), "moe_group_gemm: epilogue %d with output type %d", epilogue, y_dtype);
  GS_REQUIRE(gs_ceil_div(N, MG_BN) <= 65535, "moe_group_gemm: N=%d too wide", N);
  const size_t lds = (size_t)2 * (MG_BM + MG_BN) * MG_LDR * sizeof(uint16_t);
  dim3 grid(max_tiles, gs_ceil_div(N, MG_BN));
  if (epilogue == 0) {
    static const hipError_t asked = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_group_gemm_kernel<0, float>),
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    (void)asked;
    moe_group_gemm_kernel<0, float><<<grid, 256, lds, stream>>>((const bf16*)X, ldx, gather, (const bf16*)W, (float*)Y, ldy,
                                                               tiles, max_tiles, n_tiles, N, K);
  } else if (epilogue == 1) {
    static const hipError_t asked = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_group_gemm_kernel<1, bf16>),
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    (void)asked;
    moe_group_gemm_kernel<1, bf16><<<grid, 256, lds, stream>>>((const bf16*)X, ldx, gather, (const bf16*)W, (bf16*)Y, ldy,
                                                              tiles, max_tiles, n_tiles, N, K);
  } else {
    static const hipError_t asked = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_group_gemm_kernel<2, bf16>),
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    (void)asked;
    moe_group_gemm_kernel<2, bf16><<<grid, 256, lds, stream>>>((const bf16*)X, ldx, gather, (const bf16*)W, (bf16*)Y, ldy,
                                                              tiles, max_tiles, n_tiles, N, K);
  }
  GS_LAUNCH_CHECK("moe_group_gemm");
  return 0;
}

extern "C" int gs_moe_combine(const float* ys, const int* place_of, int top, const void* shared, const void* gate,
                              int ldg, void* y, int dtype, int T, int H, hipStream_t stream) {
  GS_REQUIRE(T >= 0 && top > 0 && H > 0, "moe_combine: bad sizes T=%d top=%d H=%d", T, top, H);
  GS_REQUIRE((shared == nullptr) == (gate == nullptr), "moe_combine: a shared expert's rows come with their gate");
  if (T == 0) return 0;
  if (dtype == GS_BF16)
    moe_combine_kernel<bf16><<<T, 256, 0, stream>>>(ys, place_of, top, (const bf16*)shared, (const bf16*)gate, ldg, (bf16*)y, H);
  else if (dtype == GS_F32)
    moe_combine_kernel<float><<<T, 256, 0, stream>>>(ys, place_of, top, (const float*)shared, (const float*)gate, ldg, (float*)y, H);
  else
    GS_REQUIRE(false, "moe_combine: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("moe_combine");
  return 0;
}
