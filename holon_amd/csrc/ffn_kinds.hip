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

// One block a row: y = a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over the row.
template <typename T, int REGS>
__global__ void __launch_bounds__(256) polynorm_kernel(const T* __restrict__ z, const float* __restrict__ coef,
                                                       T* __restrict__ y, int dim, float eps) {
  __shared__ float part[3][4];
  const int64_t base = (int64_t)blockIdx.x * dim;
  float held[REGS > 0 ? REGS : 1];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  auto take = [&](float v) { const float q = v * v; s2 += q; s4 += q * q; s6 += q * q * q; };
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = threadIdx.x + e * 256;
      held[e] = i < dim ? Elem<T>::load(z[base + i]) : 0.f;
      take(held[e]);
    }
  } else {
    for (int i = threadIdx.x; i < dim; i += 256) take(Elem<T>::load(z[base + i]));
  }
  block_sum3_256(s2, s4, s6, part);
  const float n = (float)dim;
  const float r1 = coef[0] / sqrtf(s2 / n + eps), r2 = coef[1] / sqrtf(s4 / n + eps), r3 = coef[2] / sqrtf(s6 / n + eps);
  const float e0 = coef[3];
  auto emit = [&](int i, float v) { y[base + i] = Elem<T>::store(((r1 * v + r2 * (v * v)) + r3 * (v * v * v)) + e0); };
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = threadIdx.x + e * 256;
      if (i < dim) emit(i, held[e]);
    }
  } else {
    for (int i = threadIdx.x; i < dim; i += 256) emit(i, Elem<T>::load(z[base + i]));
  }
}

#define ROUTE_MAX_E 1024

// One block of 64 threads a token. s = sigmoid(logit); choice = s + correction; groups of neighbours are ranked by the
// sum of their two largest choices and the `keep` best stay open; the `top` largest open choices are chosen (equal
// ones: the lower index first); weight = s * scale for a chosen expert, 0 for every other.
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
  if (groups > 1) {
    const int size = experts / groups;
    for (int g = threadIdx.x; g < groups; g += 64) {
      float a = -INFINITY, b = -INFINITY;                // the two largest of the group
      for (int i = 0; i < size; ++i) {
        const float v = choice_s[g * size + i];
        if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
      }
      group_s[g] = size > 1 ? a + b : a;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += 64) {
      const int g = e / size;
      const float mine = group_s[g];
      int ahead = 0;
      for (int o = 0; o < groups; ++o) ahead += (group_s[o] > mine) || (group_s[o] == mine && o < g);
      if (ahead >= keep) choice_s[e] = -INFINITY;
    }
    __syncthreads();
  }
  for (int e = threadIdx.x; e < experts; e += 64) {
    const float mine = choice_s[e];
    int ahead = 0;
    for (int o = 0; o < experts; ++o) ahead += (choice_s[o] > mine) || (choice_s[o] == mine && o < e);
    weights[base + e] = (ahead < top && mine > -INFINITY) ? score_s[e] * scale : 0.f;
  }
}

// y[t, c] = round(round(silu(gate)) * up) * weight of the column's expert, 0 where that weight is 0; columns from
// experts * ff on belong to an expert every token uses with weight 1.
template <typename T>
__global__ void __launch_bounds__(256) moe_gate_kernel(const T* __restrict__ gate_up, const float* __restrict__ weights,
                                                       T* __restrict__ y, int experts, int ff, int shared) {
  const int cols = experts * ff + shared;
  const int64_t t = blockIdx.y;
  const T* row = gate_up + t * 2 * cols;
  for (int c = blockIdx.x * 256 + threadIdx.x; c < cols; c += gridDim.x * 256) {
    const float w = c < experts * ff ? weights[t * experts + c / ff] : 1.0f;
    float out = 0.f;
    if (w != 0.f) {
      const float g = Elem<T>::load(row[c]), u = Elem<T>::load(row[cols + c]);
      out = Elem<T>::round(Elem<T>::round(silu<T>(g)) * u) * w;
    }
    y[t * cols + c] = Elem<T>::store(out);
  }
}
}  // namespace

extern "C" int holon_polynorm(const void* z, const float* coef, void* y, int64_t rows, int dim, float eps, int dtype,
                              void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 0x7fffffffLL && dim > 0, "polynorm: rows=%lld dim=%d", (long long)rows, dim);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
#define PN(T, R) polynorm_kernel<T, R><<<(unsigned)rows, 256, 0, s>>>((const T*)z, coef, (T*)y, dim, eps)
  if (dtype == HOLON_F32) { if (dim <= 1024) PN(float, 4); else if (dim <= 8192) PN(float, 32); else PN(float, 0); }
  else { if (dim <= 1024) PN(bf16_t, 4); else if (dim <= 8192) PN(bf16_t, 32); else PN(bf16_t, 0); }
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

extern "C" int holon_moe_gate(const void* gate_up, const float* weights, void* y, int64_t rows, int experts, int ff,
                              int shared, int dtype, void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 65535 * 1024LL && experts >= 1 && ff >= 1 && shared >= 0,
              "moe_gate: rows=%lld, %d experts of %d, %d shared columns", (long long)rows, experts, ff, shared);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int cols = experts * ff + shared;
  for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
    const int n = (int)(rows - r0 < 65535 ? rows - r0 : 65535);
    const dim3 grid((cols + 255) / 256 < 64 ? (cols + 255) / 256 : 64, n);
    if (dtype == HOLON_F32)
      moe_gate_kernel<float><<<grid, 256, 0, s>>>((const float*)gate_up + r0 * 2 * cols, weights + r0 * experts,
                                                   (float*)y + r0 * cols, experts, ff, shared);
    else
      moe_gate_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)gate_up + r0 * 2 * cols, weights + r0 * experts,
                                                    (bf16_t*)y + r0 * cols, experts, ff, shared);
  }
  HOLON_LAUNCH_OK();
  return 0;
}
