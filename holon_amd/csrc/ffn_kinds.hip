// The elementwise steps of two feed-forward kinds: the PolyNorm activation of a dense one, and the router's choice and
// the gated activation of a mixture of experts. float32 inside; sums over a row in an order its width alone decides.
#include "common.h"
#include "holon_hip.h"

namespace {

// Three sums over a block of 256 threads at once; waves are added in order.
__device__ __forceinline__ void block_sum3_256(float& a, float& b, float& c, float (*part)[4]) {
  a = wave_sum(a); b = wave_sum(b); c = wave_sum(c);
  __syncthreads();
  if (threadIdx.x % WAVE == 0) {
    const int w = threadIdx.x / WAVE;
    part[0][w] = a; part[1][w] = b; part[2][w] = c;
  }
  __syncthreads();
  a = (part[0][0] + part[0][1]) + (part[0][2] + part[0][3]);
  b = (part[1][0] + part[1][1]) + (part[1][2] + part[1][3]);
  c = (part[2][0] + part[2][1]) + (part[2][2] + part[2][3]);
}

// One block a row: y = a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over the row. A thread takes
// N neighbouring values at a time (N = 16 bytes' worth where rows allow, else 1); REGS such groups stay in registers
// between the two passes (0: the row is read again).
template <typename T, int REGS, bool VEC>
__global__ void __launch_bounds__(256) polynorm_kernel(const T* __restrict__ z, const float* __restrict__ coef,
                                                       T* __restrict__ y, int dim, float eps) {
  __shared__ float part[3][4];
  constexpr int N = VEC ? Elem<T>::kVec : 1;
  const int64_t base = (int64_t)blockIdx.x * dim;
  float held[(REGS > 0 ? REGS : 1) * N];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  auto take = [&](float v) { const float q = v * v; s2 += q; s4 += q * q; s6 += q * q * q; };
  auto load = [&](int i, float* to) {                    // N values from column i on
    if constexpr (VEC) {
      const uint4 raw = *reinterpret_cast<const uint4*>(z + base + i);
      const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
      for (int u = 0; u < N; ++u) to[u] = Elem<T>::load(e[u]);
    } else {
      to[0] = Elem<T>::load(z[base + i]);
    }
  };
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = (threadIdx.x + e * 256) * N;
      if (i < dim) load(i, held + e * N);
      else
#pragma unroll
        for (int u = 0; u < N; ++u) held[e * N + u] = 0.f;
#pragma unroll
      for (int u = 0; u < N; ++u) take(held[e * N + u]);
    }
  } else {
    for (int i = threadIdx.x * N; i < dim; i += 256 * N) {
      load(i, held);
#pragma unroll
      for (int u = 0; u < N; ++u) take(held[u]);
    }
  }
  block_sum3_256(s2, s4, s6, part);
  const float n = (float)dim;
  const float r1 = coef[0] / sqrtf(s2 / n + eps), r2 = coef[1] / sqrtf(s4 / n + eps), r3 = coef[2] / sqrtf(s6 / n + eps);
  const float e0 = coef[3];
  auto emit = [&](int i, const float* v) {
    if constexpr (VEC) {
      uint4 out;
      T* o = reinterpret_cast<T*>(&out);
#pragma unroll
      for (int u = 0; u < N; ++u) o[u] = Elem<T>::store(((r1 * v[u] + r2 * (v[u] * v[u])) + r3 * (v[u] * v[u] * v[u])) + e0);
      *reinterpret_cast<uint4*>(y + base + i) = out;
    } else {
      y[base + i] = Elem<T>::store(((r1 * v[0] + r2 * (v[0] * v[0])) + r3 * (v[0] * v[0] * v[0])) + e0);
    }
  };
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = (threadIdx.x + e * 256) * N;
      if (i < dim) emit(i, held + e * N);
    }
  } else {
    for (int i = threadIdx.x * N; i < dim; i += 256 * N) {
      load(i, held);
      emit(i, held);
    }
  }
}

#define ROUTE_MAX_E 1024

// The router's choice for one token, by all threads of a block: score_s holds s = sigmoid(logit), choice_s the choice
// scores s + correction. Groups of neighbours are ranked by the sum of their two largest choices and the `keep` best
// stay open; the `top` largest open choices are chosen (equal ones: the lower index first); weight = s * scale for a
// chosen expert, 0 for every other.
__device__ __forceinline__ void route_token(float* score_s, float* choice_s, float* group_s, float* __restrict__ weights,
                                            int experts, int top, int groups, int keep, float scale) {
  const int step = blockDim.x;
  if (groups > 1) {
    const int size = experts / groups;
    for (int g = threadIdx.x; g < groups; g += step) {
      float a = -INFINITY, b = -INFINITY;                // the two largest of the group
      for (int i = 0; i < size; ++i) {
        const float v = choice_s[g * size + i];
        if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
      }
      group_s[g] = size > 1 ? a + b : a;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += step) {
      const int g = e / size;
      const float mine = group_s[g];
      int ahead = 0;
      for (int o = 0; o < groups; ++o) ahead += (group_s[o] > mine) || (group_s[o] == mine && o < g);
      if (ahead >= keep) choice_s[e] = -INFINITY;
    }
    __syncthreads();
  }
  for (int e = threadIdx.x; e < experts; e += step) {
    const float mine = choice_s[e];
    int ahead = 0;
    for (int o = 0; o < experts; ++o) ahead += (choice_s[o] > mine) || (choice_s[o] == mine && o < e);
    weights[e] = (ahead < top && mine > -INFINITY) ? score_s[e] * scale : 0.f;
  }
}

// One block of 64 threads a token, from logits.
__global__ void __launch_bounds__(64) moe_route_kernel(const float* __restrict__ logits,
                                                       const float* __restrict__ correction, float* __restrict__ weights,
                                                       int experts, int top, int groups, int keep, float scale) {
  __shared__ float score_s[ROUTE_MAX_E];
  __shared__ float choice_s[ROUTE_MAX_E];
  __shared__ float group_s[ROUTE_MAX_E];
  const int64_t base = (int64_t)blockIdx.x * experts;
  for (int e = threadIdx.x; e < experts; e += 64) {
    const float s = 1.0f / (1.0f + expf(-logits[base + e]));
    score_s[e] = s;
    choice_s[e] = correction ? s + correction[e] : s;
  }
  __syncthreads();
  route_token(score_s, choice_s, group_s, weights + base, experts, top, groups, keep, scale);
}

// One block of 256 threads a token, from the token's row: the float32 logits x . router[e] first (the row waits in LDS
// as float32; wave w takes experts w, w + 4, ..., its lanes a 64th of the row each, added up in an order the width
// alone decides), then the choice.
template <typename T>
__global__ void __launch_bounds__(256) moe_router_kernel(const T* __restrict__ x, const float* __restrict__ router,
                                                         const float* __restrict__ correction,
                                                         float* __restrict__ weights, int width, int experts, int top,
                                                         int groups, int keep, float scale) {
  extern __shared__ float xs[];                          // [width]
  __shared__ float score_s[ROUTE_MAX_E];
  __shared__ float choice_s[ROUTE_MAX_E];
  __shared__ float group_s[ROUTE_MAX_E];
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < width; i += 256) xs[i] = Elem<T>::load(x[t * width + i]);
  __syncthreads();
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const bool wide = width % 4 == 0 && (uintptr_t)router % 16 == 0;
  for (int e = wave; e < experts; e += 4) {
    const float* w = router + (int64_t)e * width;
    float acc = 0.f;
    if (wide) {
      for (int i = lane * 4; i < width; i += WAVE * 4) {
        const float4 v = *reinterpret_cast<const float4*>(w + i);
        acc += xs[i] * v.x + xs[i + 1] * v.y + xs[i + 2] * v.z + xs[i + 3] * v.w;
      }
    } else {
      for (int i = lane; i < width; i += WAVE) acc += xs[i] * w[i];
    }
    acc = wave_sum(acc);
    if (lane == 0) {
      const float s = 1.0f / (1.0f + expf(-acc));
      score_s[e] = s;
      choice_s[e] = correction ? s + correction[e] : s;
    }
  }
  __syncthreads();
  route_token(score_s, choice_s, group_s, weights + t * experts, experts, top, groups, keep, scale);
}

// y[t, c] = round(round(silu(gate)) * up) * weight of the column's expert, 0 where that weight is 0; columns from
// experts * ff on belong to an expert every token uses with weight 1, or with the weight in column `shared_col` of the
// weights' rows (which are `wstride` long). VEC: a thread takes 16 bytes of a row at a time
// (every row and the border between gates and ups fall on 16 bytes, and a group of columns is one expert's).
template <typename T, bool VEC>
__global__ void __launch_bounds__(256) moe_gate_kernel(const T* __restrict__ gate_up, const float* __restrict__ weights,
                                                       T* __restrict__ y, int experts, int ff, int shared,
                                                       int wstride, int shared_col) {
  const int cols = experts * ff + shared;
  const int64_t t = blockIdx.y;
  const T* row = gate_up + t * 2 * cols;
  constexpr int N = VEC ? Elem<T>::kVec : 1;
  for (int c = (blockIdx.x * 256 + threadIdx.x) * N; c < cols; c += gridDim.x * 256 * N) {
    const float w = c < experts * ff ? weights[t * wstride + c / ff]
                                     : (shared_col >= 0 ? weights[t * wstride + shared_col] : 1.0f);
    if constexpr (VEC) {
      uint4 out = make_uint4(0u, 0u, 0u, 0u);
      if (w != 0.f) {
        const uint4 graw = *reinterpret_cast<const uint4*>(row + c), uraw = *reinterpret_cast<const uint4*>(row + cols + c);
        const T* g = reinterpret_cast<const T*>(&graw);
        const T* u = reinterpret_cast<const T*>(&uraw);
        T* o = reinterpret_cast<T*>(&out);
#pragma unroll
        for (int i = 0; i < N; ++i)
          o[i] = Elem<T>::store(Elem<T>::round(Elem<T>::round(silu<T>(Elem<T>::load(g[i]))) * Elem<T>::load(u[i])) * w);
      }
      *reinterpret_cast<uint4*>(y + t * cols + c) = out;
    } else {
      float out = 0.f;
      if (w != 0.f) {
        const float g = Elem<T>::load(row[c]), u = Elem<T>::load(row[cols + c]);
        out = Elem<T>::round(Elem<T>::round(silu<T>(g)) * u) * w;
      }
      y[t * cols + c] = Elem<T>::store(out);
    }
  }
}
// The other router, one block of 256 threads a token: float32 logits z_e = x . router[e] + bias[e]; the `top` largest
// are chosen (equal ones: the lower index first) and weighted by the softmax over the chosen logits alone, every other
// expert 0. Rows of `router` beyond the experts are gates: their columns hold sigmoid(x . router[r]).
// Every thread takes a slice of the token's row against all router rows, sixteen rows at a time (their loads do not
// wait for each other); a wave's lanes are summed by shuffles and the four waves' partial sums in wave order. Up to 64
// experts one wave then makes the choice with an expert a lane; more are ranked by the whole block.
template <typename T>
__global__ void __launch_bounds__(256) moe_router_top_kernel(const T* __restrict__ x, const float* __restrict__ router,
                                                             const float* __restrict__ bias, float* __restrict__ weights,
                                                             int width, int experts, int rows_r, int top) {
  __shared__ float part_s[4][ROUTE_MAX_E + 1];
  __shared__ float z_s[ROUTE_MAX_E + 1];
  __shared__ float e_s[ROUTE_MAX_E];
  __shared__ float red_s[4];
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* row = x + t * width;
  const bool wide = width % 4 == 0 && (uintptr_t)router % 16 == 0 && (uintptr_t)x % 16 == 0;
  for (int e0 = 0; e0 < rows_r; e0 += 16) {
    float acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0.f;
    if (wide) {
      for (int i = threadIdx.x * 4; i < width; i += 1024) {
        const float x0 = Elem<T>::load(row[i]), x1 = Elem<T>::load(row[i + 1]), x2 = Elem<T>::load(row[i + 2]),
                    x3 = Elem<T>::load(row[i + 3]);
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          if (e0 + j < rows_r) {
            const float4 v = *reinterpret_cast<const float4*>(router + (int64_t)(e0 + j) * width + i);
            acc[j] += x0 * v.x + x1 * v.y + x2 * v.z + x3 * v.w;
          }
        }
      }
    } else {
      for (int i = threadIdx.x; i < width; i += 256) {
        const float xv = Elem<T>::load(row[i]);
#pragma unroll
        for (int j = 0; j < 16; ++j)
          if (e0 + j < rows_r) acc[j] += xv * router[(int64_t)(e0 + j) * width + i];
      }
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      if (e0 + j < rows_r) {
        const float a = wave_sum(acc[j]);
        if (lane == 0) part_s[wave][e0 + j] = a;
      }
    }
  }
  __syncthreads();
  auto logit = [&](int e) {
    const float z = ((part_s[0][e] + part_s[1][e]) + part_s[2][e]) + part_s[3][e];
    return e < experts && bias ? z + bias[e] : z;
  };
  if (experts <= WAVE) {                                  // an expert a lane
    if (wave != 0) return;
    const float mine = lane < experts ? logit(lane) : -INFINITY;
    int ahead = 0;
    for (int o = 0; o < experts; ++o) {
      const float other = __shfl(mine, o, WAVE);
      ahead += (other > mine) || (other == mine && o < lane);
    }
    const float top_z = wave_max(mine);                   // the largest logit is always chosen
    const float v = lane < experts && ahead < top ? expf(mine - top_z) : 0.f;
    const float sum = wave_sum(v);
    if (lane < experts) weights[t * rows_r + lane] = v / sum;
    if (rows_r > experts && lane == 0) weights[t * rows_r + experts] = 1.0f / (1.0f + expf(-logit(experts)));
    return;
  }
  for (int e = threadIdx.x; e < rows_r; e += 256) z_s[e] = logit(e);
  __syncthreads();
  float top_z = -INFINITY;
  for (int e = threadIdx.x; e < experts; e += 256) top_z = fmaxf(top_z, z_s[e]);
  top_z = wave_max(top_z);
  if (lane == 0) red_s[wave] = top_z;
  __syncthreads();
  top_z = fmaxf(fmaxf(red_s[0], red_s[1]), fmaxf(red_s[2], red_s[3]));
  __syncthreads();
  float part = 0.f;
  for (int e = threadIdx.x; e < experts; e += 256) {
    const float mine = z_s[e];
    int ahead = 0;
    for (int o = 0; o < experts; ++o) ahead += (z_s[o] > mine) || (z_s[o] == mine && o < e);
    const float v = ahead < top ? expf(mine - top_z) : 0.f;
    e_s[e] = v;
    part += v;
  }
  part = wave_sum(part);
  if (lane == 0) red_s[wave] = part;
  __syncthreads();
  const float sum = ((red_s[0] + red_s[1]) + red_s[2]) + red_s[3];
  for (int e = threadIdx.x; e < rows_r; e += 256)
    weights[t * rows_r + e] = e < experts ? e_s[e] / sum : 1.0f / (1.0f + expf(-z_s[e]));
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(256) relu2_kernel(const T* __restrict__ z, T* __restrict__ y, int64_t n) {
  constexpr int N = VEC ? Elem<T>::kVec : 1;
  for (int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * N; i < n; i += (int64_t)gridDim.x * 256 * N) {
    if constexpr (VEC) {
      const uint4 raw = *reinterpret_cast<const uint4*>(z + i);
      const T* in = reinterpret_cast<const T*>(&raw);
      uint4 out;
      T* o = reinterpret_cast<T*>(&out);
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const float v = fmaxf(Elem<T>::load(in[j]), 0.f);
        o[j] = Elem<T>::store(v * v);
      }
      *reinterpret_cast<uint4*>(y + i) = out;
    } else {
      const float v = fmaxf(Elem<T>::load(z[i]), 0.f);
      y[i] = Elem<T>::store(v * v);
    }
  }
}
}  // namespace

extern "C" int holon_polynorm(const void* z, const float* coef, void* y, int64_t rows, int dim, float eps, int dtype,
                              void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 0x7fffffffLL && dim > 0, "polynorm: rows=%lld dim=%d", (long long)rows, dim);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  // in groups of 16 bytes where every row starts on such a border; the sums then run in another order than value by
  // value, but still in one that the width alone decides
  const int vec = dtype == HOLON_F32 ? 4 : 8;
  const bool wide = dim % vec == 0 && (uintptr_t)z % 16 == 0 && (uintptr_t)y % 16 == 0;
  const int groups = wide ? dim / vec : dim;
#define PN(T, R, V) polynorm_kernel<T, R, V><<<(unsigned)rows, 256, 0, s>>>((const T*)z, coef, (T*)y, dim, eps)
#define PN_BY_SIZE(T, V)                      \
  do {                                        \
    if (groups <= 256) PN(T, 1, V);           \
    else if (groups <= 1024) PN(T, 4, V);     \
    else if (!V && groups <= 4096) PN(T, 16, V); \
    else PN(T, 0, V);                         \
  } while (0)
  if (dtype == HOLON_F32) { if (wide) PN_BY_SIZE(float, true); else PN_BY_SIZE(float, false); }
  else { if (wide) PN_BY_SIZE(bf16_t, true); else PN_BY_SIZE(bf16_t, false); }
#undef PN_BY_SIZE
#undef PN
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_moe_route(const float* logits, const float* correction, float* weights, int64_t rows, int experts,
                               int top, int groups, int keep, float scale, void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 0x7fffffffLL && experts >= 1 && experts <= ROUTE_MAX_E && top >= 1 && top <= experts,
              "moe_route: rows=%lld, top %d of %d experts (at most %d)", (long long)rows, top, experts, ROUTE_MAX_E);
  HOLON_CHECK(groups <= 1 || (experts % groups == 0 && keep >= 1 && keep <= groups),
              "moe_route: %d experts in %d groups of which %d stay open", experts, groups, keep);
  if (rows == 0) return 0;
  moe_route_kernel<<<(unsigned)rows, 64, 0, (hipStream_t)stream>>>(logits, correction, weights, experts, top, groups,
                                                                    keep, scale);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_moe_router(const void* x, const float* router, const float* correction, float* weights,
                                int64_t rows, int width, int experts, int top, int groups, int keep, float scale,
                                int dtype, void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 0x7fffffffLL && width >= 1 && width <= 12288 && experts >= 1 &&
                  experts <= ROUTE_MAX_E && top >= 1 && top <= experts,
              "moe_router: rows=%lld of %d (at most 12,288), top %d of %d experts (at most %d)", (long long)rows, width,
              top, experts, ROUTE_MAX_E);
  HOLON_CHECK(groups <= 1 || (experts % groups == 0 && keep >= 1 && keep <= groups),
              "moe_router: %d experts in %d groups of which %d stay open", experts, groups, keep);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)width * sizeof(float);
  if (dtype == HOLON_F32)
    moe_router_kernel<float><<<(unsigned)rows, 256, lds, s>>>((const float*)x, router, correction, weights, width,
                                                             experts, top, groups, keep, scale);
  else
    moe_router_kernel<bf16_t><<<(unsigned)rows, 256, lds, s>>>((const bf16_t*)x, router, correction, weights, width,
                                                              experts, top, groups, keep, scale);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_moe_gate(const void* gate_up, const float* weights, void* y, int64_t rows, int experts, int ff,
                              int shared, int dtype, int wstride, int shared_col, void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 65535 * 1024LL && experts >= 1 && ff >= 1 && shared >= 0,
              "moe_gate: rows=%lld, %d experts of %d, %d shared columns", (long long)rows, experts, ff, shared);
  HOLON_CHECK(wstride >= experts && shared_col < wstride, "moe_gate: weight rows of %d for %d experts, column %d",
              wstride, experts, shared_col);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int cols = experts * ff + shared;
  for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
    const int n = (int)(rows - r0 < 65535 ? rows - r0 : 65535);
    const int vec = dtype == HOLON_F32 ? 4 : 8;
    const bool wide = ff % vec == 0 && shared % vec == 0 && (uintptr_t)gate_up % 16 == 0 && (uintptr_t)y % 16 == 0;
    const int groups = wide ? cols / vec : cols;
    const dim3 grid((groups + 255) / 256 < 64 ? (groups + 255) / 256 : 64, n);
#define MOE_GATE(T, V)                                                                                        \
  moe_gate_kernel<T, V><<<grid, 256, 0, s>>>((const T*)gate_up + r0 * 2 * cols, weights + r0 * wstride,       \
                                             (T*)y + r0 * cols, experts, ff, shared, wstride, shared_col)
    if (dtype == HOLON_F32) { if (wide) MOE_GATE(float, true); else MOE_GATE(float, false); }
    else { if (wide) MOE_GATE(bf16_t, true); else MOE_GATE(bf16_t, false); }
#undef MOE_GATE
  }
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_moe_router_top(const void* x, const float* router, const float* bias, float* weights, int64_t rows,
                                    int width, int experts, int router_rows, int top, int dtype, void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 0x7fffffffLL && width >= 1 && width <= 12288 && experts >= 1 &&
                  experts <= ROUTE_MAX_E && top >= 1 && top <= experts &&
                  (router_rows == experts || router_rows == experts + 1),
              "moe_router_top: rows=%lld of %d (at most 12,288), top %d of %d experts (at most %d), %d router rows",
              (long long)rows, width, top, experts, ROUTE_MAX_E, router_rows);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    moe_router_top_kernel<float><<<(unsigned)rows, 256, 0, s>>>((const float*)x, router, bias, weights, width, experts,
                                                               router_rows, top);
  else
    moe_router_top_kernel<bf16_t><<<(unsigned)rows, 256, 0, s>>>((const bf16_t*)x, router, bias, weights, width,
                                                                experts, router_rows, top);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_relu2(const void* z, void* y, int64_t n, int dtype, void* stream) {
  HOLON_CHECK(n >= 0, "relu2: n=%lld", (long long)n);
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int vec = dtype == HOLON_F32 ? 4 : 8;
  const bool wide = n % vec == 0 && (uintptr_t)z % 16 == 0 && (uintptr_t)y % 16 == 0;
  const int64_t groups = wide ? n / vec : n;
  const unsigned blocks = (unsigned)((groups + 255) / 256 < 16384 ? (groups + 255) / 256 : 16384);
  if (dtype == HOLON_F32) {
    if (wide) relu2_kernel<float, true><<<blocks, 256, 0, s>>>((const float*)z, (float*)y, n);
    else relu2_kernel<float, false><<<blocks, 256, 0, s>>>((const float*)z, (float*)y, n);
  } else {
    if (wide) relu2_kernel<bf16_t, true><<<blocks, 256, 0, s>>>((const bf16_t*)z, (bf16_t*)y, n);
    else relu2_kernel<bf16_t, false><<<blocks, 256, 0, s>>>((const bf16_t*)z, (bf16_t*)y, n);
  }
  HOLON_LAUNCH_OK();
  return 0;
}
