// The kernels of a block whose two sublayers read the same float32 residual stream: one pass over a row adds what the
// layer before left to add (two terms, summed first) and a vector of the pass that begins, takes the row's mean square
// once and writes the row normed with one weight or with two. Every sum over a row is taken in an order that the row's
// width alone decides, so a token's result does not depend on what else is in the batch.
#include "common.h"
#include "holon_hip.h"

namespace {

__device__ __forceinline__ float load_as(const void* p, int64_t i, int dt) {
  return dt == HOLON_F32 ? reinterpret_cast<const float*>(p)[i] : bf16_to_float(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void store_as(void* p, int64_t i, int dt, float v) {
  if (dt == HOLON_F32) reinterpret_cast<float*>(p)[i] = v;
  else reinterpret_cast<bf16_t*>(p)[i] = float_to_bf16(v);
}

// Sum over a block of 256 threads, every thread gets the result; waves are added in order.
__device__ __forceinline__ float block_sum_256(float v, float* part) {
  v = wave_sum(v);
  __syncthreads();
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = v;
  __syncthreads();
  return (part[0] + part[1]) + (part[2] + part[3]);
}

// One block a row. REGS: the row (up to 256 * REGS values) stays in registers between the two passes; 0: it is read
// back from memory (a thread reads what it wrote itself).
template <int REGS>
__global__ void __launch_bounds__(256) stream_rms_kernel(float* __restrict__ x32, const void* __restrict__ d1, int dt1,
                                                         const void* __restrict__ d2, int dt2,
                                                         const float* __restrict__ row, const void* __restrict__ w1,
                                                         const void* __restrict__ w2, int dtw, void* __restrict__ y1,
                                                         void* __restrict__ y2, int dim, float eps, int dt_out) {
  __shared__ float part[4];
  const int64_t base = (int64_t)blockIdx.x * dim;
  float* x = x32 + base;
  float held[REGS > 0 ? REGS : 1];
  float sq = 0.f;
  auto updated = [&](int i) {
    float v = x[i];
    if (d1) {
      float a = load_as(d1, base + i, dt1);
      if (d2) a += load_as(d2, base + i, dt2);
      v += a;
    }
    if (row) v += row[i];
    if (d1 || row) x[i] = v;
    return v;
  };
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = threadIdx.x + e * 256;
      held[e] = i < dim ? updated(i) : 0.f;
      sq += held[e] * held[e];
    }
  } else {
    for (int i = threadIdx.x; i < dim; i += 256) { const float v = updated(i); sq += v * v; }
  }
  if (!w1) return;
  sq = block_sum_256(sq, part);
  const float r = 1.0f / sqrtf(sq / (float)dim + eps);
  auto emit = [&](int i, float v) {
    const float u = v * r;
    store_as(y1, base + i, dt_out, u * load_as(w1, i, dtw));
    if (w2) store_as(y2, base + i, dt_out, u * load_as(w2, i, dtw));
  };
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = threadIdx.x + e * 256;
      if (i < dim) emit(i, held[e]);
    }
  } else {
    for (int i = threadIdx.x; i < dim; i += 256) emit(i, x[i]);
  }
}

__global__ void scale_rows_kernel(const void* __restrict__ x, float* __restrict__ y, int64_t n, int dt, float scale) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    y[i] = load_as(x, i, dt) * scale;
}
}  // namespace

extern "C" int holon_stream_rms(float* x32, const void* d1, int dt1, const void* d2, int dt2, const float* row,
                                const void* w1, const void* w2, int dtw, void* y1, void* y2, int64_t rows, int dim,
                                float eps, int dt_out, void* stream) {
  HOLON_CHECK(rows >= 0 && dim > 0 && rows <= 0x7fffffffLL, "stream_rms: rows=%lld dim=%d", (long long)rows, dim);
  HOLON_CHECK((w1 == nullptr) == (y1 == nullptr) && (w2 == nullptr) == (y2 == nullptr) && (w1 != nullptr || w2 == nullptr),
              "stream_rms: a weight comes with its result, the second only beside the first");
  HOLON_CHECK(d1 != nullptr || d2 == nullptr, "stream_rms: a second term without the first");
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
#define SRMS(R) stream_rms_kernel<R><<<(unsigned)rows, 256, 0, s>>>(x32, d1, dt1, d2, dt2, row, w1, w2, dtw, y1, y2, dim, eps, dt_out)
  if (dim <= 1024) SRMS(4);
  else if (dim <= 4096) SRMS(16);
  else SRMS(0);
#undef SRMS
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_scale_rows(const void* x, float* y, int64_t n, int dtype, float scale, void* stream) {
  HOLON_CHECK(n >= 0 && (dtype == HOLON_F32 || dtype == HOLON_BF16), "scale_rows: n=%lld dtype=%d", (long long)n, dtype);
  if (n == 0) return 0;
  const int64_t blocks = (n + 255) / 256;
  scale_rows_kernel<<<(unsigned)(blocks < 4096 ? blocks : 4096), 256, 0, (hipStream_t)stream>>>(x, y, n, dtype, scale);
  HOLON_LAUNCH_OK();
  return 0;
}
