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

// Four neighbouring values at a time.
__device__ __forceinline__ void load4(const void* p, int64_t i, int dt, float (&v)[4]) {
  if (dt == HOLON_F32) {
    const float4 f = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i);
    v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
  } else {
    const ushort4 h = *reinterpret_cast<const ushort4*>(reinterpret_cast<const bf16_t*>(p) + i);
    v[0] = bf16_to_float(h.x); v[1] = bf16_to_float(h.y); v[2] = bf16_to_float(h.z); v[3] = bf16_to_float(h.w);
  }
}
__device__ __forceinline__ void store4(void* p, int64_t i, int dt, const float (&v)[4]) {
  if (dt == HOLON_F32) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(p) + i) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    ushort4 h;
    h.x = float_to_bf16(v[0]); h.y = float_to_bf16(v[1]); h.z = float_to_bf16(v[2]); h.w = float_to_bf16(v[3]);
    *reinterpret_cast<ushort4*>(reinterpret_cast<bf16_t*>(p) + i) = h;
  }
}
// The same with the element type known when the kernel is compiled (a branch on the type around every load keeps the
// loads from being under way together).
template <int DT>
__device__ __forceinline__ void load4t(const void* p, int64_t i, float (&v)[4]) { load4(p, i, DT, v); }
template <int DT>
__device__ __forceinline__ void store4t(void* p, int64_t i, const float (&v)[4]) { store4(p, i, DT, v); }
__device__ __forceinline__ float rounded(float v, int dt) { return dt == HOLON_F32 ? v : bf16_to_float(float_to_bf16(v)); }

// What the filters of a step of single tokens need (row b is token b): the taps [dim, taps] of the two filters (the
// second nullable), the requests' last taps - 1 inputs of each [slots, taps - 1, dim], all of the results' dtype.
struct Filters {
  const void* w1;
  const void* w2;
  void* held1;
  void* held2;
  const int32_t* slots;
  const int32_t* starts;
  int taps;
};

// y <- a + sum_j w[c, j] a_(t - taps + 1 + j), for a row's single token whose earlier inputs wait in its slot (zeros
// for a row that starts its sequence): taps added oldest first in float32, then the input, one rounding; the slot
// then holds the last taps - 1 inputs with this one at their end. `a`: the rounded inputs of channels c0 .. c0 + 3.
// Everything is read before anything is written (a store in between would make every later load wait for it).
template <int TAPS, int DT>
struct Filter4 {
  float old[TAPS > 1 ? TAPS - 1 : 1][4];
  float taps[TAPS][4];                                   // the four channels' taps as they lie: [channel][tap] flat
  int64_t base;
  __device__ __forceinline__ void load(const void* held, const void* w, int slot, bool carried, int c0, int dim) {
    base = (int64_t)slot * (TAPS - 1) * dim + c0;
#pragma unroll
    for (int j = 0; j + 1 < TAPS; ++j) {                   // (a slot that is not carried is read all the same, and
      load4t<DT>(held, base + (int64_t)j * dim, old[j]);   // what it held counts as zeros)
      if (!carried) old[j][0] = old[j][1] = old[j][2] = old[j][3] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < TAPS; ++j) load4t<DT>(w, (int64_t)c0 * TAPS + 4 * j, taps[j]);
  }
  __device__ __forceinline__ void apply(const float (&a)[4], float (&y)[4]) const {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j + 1 < TAPS; ++j) acc += taps[(u * TAPS + j) / 4][(u * TAPS + j) % 4] * old[j][u];
      acc += taps[(u * TAPS + TAPS - 1) / 4][(u * TAPS + TAPS - 1) % 4] * a[u];
      y[u] = acc + a[u];
    }
  }
  __device__ __forceinline__ void keep(void* held, const float (&a)[4], int dim) const {
#pragma unroll
    for (int j = 1; j + 1 < TAPS; ++j) store4t<DT>(held, base + (int64_t)(j - 1) * dim, old[j]);
    if (TAPS > 1) store4t<DT>(held, base + (int64_t)(TAPS - 2) * dim, a);
  }
};

// The same pass as stream_rms_kernel with four neighbouring values a thread and step (dim a multiple of 4, at most
// 1024 REGS values a row, which stay in registers). FILTER: the step's rows are single tokens, and each result goes
// through its causal filter of TAPS taps before it is stored (see `filter4`).
template <int REGS, int TAPS, int DT = HOLON_BF16>     // DT: the results' (and the filters') dtype, read when TAPS > 0
__global__ void __launch_bounds__(256) stream_rms_vec_kernel(float* __restrict__ x32, const void* __restrict__ d1, int dt1,
                                                             const void* __restrict__ d2, int dt2,
                                                             const float* __restrict__ row, const void* __restrict__ w1,
                                                             const void* __restrict__ w2, int dtw, void* __restrict__ y1,
                                                             void* __restrict__ y2, int dim, float eps, int dt_out,
                                                             Filters f) {
  __shared__ float part[4];
  const int64_t base = (int64_t)blockIdx.x * dim;
  float held[REGS][4];
  float sq = 0.f;
#pragma unroll
  for (int e = 0; e < REGS; ++e) {
    const int i = (threadIdx.x + e * 256) * 4;
    float (&v)[4] = held[e];
    v[0] = v[1] = v[2] = v[3] = 0.f;
    if (i < dim) {
      load4(x32, base + i, HOLON_F32, v);
      if (d1) {
        float a[4];
        load4(d1, base + i, dt1, a);
        if (d2) {
          float b[4];
          load4(d2, base + i, dt2, b);
#pragma unroll
          for (int u = 0; u < 4; ++u) a[u] += b[u];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] += a[u];
      }
      if (row) {
        float b[4];
        load4(row, i, HOLON_F32, b);
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] += b[u];
      }
      if (d1 || row) store4(x32, base + i, HOLON_F32, v);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) sq += v[u] * v[u];
  }
  if (!w1) return;
  constexpr bool FILTER = TAPS > 0;
  // the filters' old inputs and taps are asked for now, so that they arrive while the row's sum is taken
  Filter4<FILTER ? TAPS : 1, DT> f1[FILTER ? REGS : 1], f2[FILTER ? REGS : 1];
  if constexpr (FILTER) {
    const int slot = f.slots[blockIdx.x];
    const bool carried = f.starts[blockIdx.x] > 0;
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = (threadIdx.x + e * 256) * 4;
      if (i >= dim) continue;
      f1[e].load(f.held1, f.w1, slot, carried, i, dim);
      if (w2) f2[e].load(f.held2, f.w2, slot, carried, i, dim);
    }
  }
  sq = block_sum_256(sq, part);
  const float r = 1.0f / sqrtf(sq / (float)dim + eps);
#pragma unroll
  for (int e = 0; e < REGS; ++e) {
    const int i = (threadIdx.x + e * 256) * 4;
    if (i >= dim) continue;
    float g[4], y[4], z[4];
    load4(w1, i, dtw, g);
#pragma unroll
    for (int u = 0; u < 4; ++u) y[u] = held[e][u] * r * g[u];
    if (w2) {
      load4(w2, i, dtw, g);
#pragma unroll
      for (int u = 0; u < 4; ++u) z[u] = held[e][u] * r * g[u];
    }
    if constexpr (FILTER) {
      float a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) { a[u] = rounded(y[u], dt_out); b[u] = w2 ? rounded(z[u], dt_out) : 0.f; }
      f1[e].apply(a, y);
      if (w2) f2[e].apply(b, z);
      f1[e].keep(f.held1, a, dim);
      if (w2) f2[e].keep(f.held2, b, dim);
    }
    store4(y1, base + i, dt_out, y);
    if (w2) store4(y2, base + i, dt_out, z);
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
  if (dim % 4 == 0 && dim <= 8192) {        // four values a thread and step (every operand is a tensor's start: 16 bytes)
    const Filters none{};
#define SRMSV(R) stream_rms_vec_kernel<R, 0><<<(unsigned)rows, 256, 0, s>>>(x32, d1, dt1, d2, dt2, row, w1, w2, dtw, y1, y2, dim, eps, dt_out, none)
    if (dim <= 1024) SRMSV(1);
    else if (dim <= 2048) SRMSV(2);
    else if (dim <= 4096) SRMSV(4);
    else SRMSV(8);
#undef SRMSV
    HOLON_LAUNCH_OK();
    return 0;
  }
#define SRMS(R) stream_rms_kernel<R><<<(unsigned)rows, 256, 0, s>>>(x32, d1, dt1, d2, dt2, row, w1, w2, dtw, y1, y2, dim, eps, dt_out)
  if (dim <= 1024) SRMS(4);
  else if (dim <= 4096) SRMS(16);
  else SRMS(0);
#undef SRMS
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_stream_rms_filter_supported(int dim, int taps) { return dim % 4 == 0 && dim <= 8192 && taps >= 1 && taps <= 4; }

// The same for a step whose rows are single tokens (row b is token b), with each result going through its causal filter
// (y <- y + conv(y), the request's last taps - 1 inputs in its slot, ignored by a row that starts at 0 and replaced
// afterwards): cw1, cw2 [dim, taps] and held1, held2 [slots, taps - 1, dim] of the results' dtype.
extern "C" int holon_stream_rms_filter(float* x32, const void* d1, int dt1, const void* d2, int dt2, const float* row,
                                       const void* w1, const void* w2, int dtw, void* y1, void* y2, int64_t rows,
                                       int dim, float eps, int dt_out, const void* cw1, const void* cw2, void* held1,
                                       void* held2, const int32_t* slots, const int32_t* starts, int taps,
                                       void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 0x7fffffffLL && holon_stream_rms_filter_supported(dim, taps),
              "stream_rms_filter: rows=%lld dim=%d (a multiple of 4, at most 8,192) taps=%d (1 to 4)", (long long)rows,
              dim, taps);
  HOLON_CHECK(w1 && y1 && cw1 && (taps == 1 || held1) && (w2 == nullptr) == (y2 == nullptr) &&
                  (w2 == nullptr || (cw2 && (taps == 1 || held2))) && slots && starts && (d1 != nullptr || d2 == nullptr),
              "stream_rms_filter: every result comes with its weight, its taps and its slots");
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const Filters f{cw1, cw2, held1, held2, slots, starts, taps};
#define SRMSF(R, K)                                                                                                  \
  do {                                                                                                               \
    if (dt_out == HOLON_F32)                                                                                         \
      stream_rms_vec_kernel<R, K, HOLON_F32><<<(unsigned)rows, 256, 0, s>>>(x32, d1, dt1, d2, dt2, row, w1, w2, dtw, \
                                                                            y1, y2, dim, eps, dt_out, f);            \
    else                                                                                                             \
      stream_rms_vec_kernel<R, K, HOLON_BF16><<<(unsigned)rows, 256, 0, s>>>(x32, d1, dt1, d2, dt2, row, w1, w2,     \
                                                                             dtw, y1, y2, dim, eps, dt_out, f);      \
  } while (0)
#define SRMSF_BY_TAPS(R)                                                        \
  do {                                                                          \
    if (taps == 1) SRMSF(R, 1); else if (taps == 2) SRMSF(R, 2);                \
    else if (taps == 3) SRMSF(R, 3); else SRMSF(R, 4);                          \
  } while (0)
  if (dim <= 1024) SRMSF_BY_TAPS(1);
  else if (dim <= 2048) SRMSF_BY_TAPS(2);
  else if (dim <= 4096) SRMSF_BY_TAPS(4);
  else SRMSF_BY_TAPS(8);
#undef SRMSF_BY_TAPS
#undef SRMSF
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
