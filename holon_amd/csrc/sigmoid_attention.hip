// Windowed attention with sigmoid weights over a paged cache whose keys and values may differ in width.
//
// One page of one site holds P tokens: keys [Hkv, P, D] (a token's key is a row) followed by values [Hkv, V, P]
// (transposed inside the page: a matrix-core operand of the value product is then one contiguous load; with V = D this
// is the layout of the framework's softmax attention). `head_prepare`
// norms and rotates the heads of a merged q/k/v projection and stores keys and values; `sigmoid_attention` sums
// sigmoid(q . k * scale + bias) * v over the keys a query sees. Nothing is normalised over keys, so there is no running
// maximum and no rescaling: a query's result is a plain sum, taken over its keys from the oldest visible one on, in
// tiles of 64 dealt to four waves in turn, an order that the query's position alone decides. Scores, weights and sums
// are float32.
#include "common.h"
#include "holon_hip.h"

#define SIG_MAX_D 512

namespace {

// One wave per (token, head of q, k or v). A row of `qkv` is `stride` values long and holds q, k and v in its first
// columns. `bias` (one float32 a column of q, k and v, or null) is added first. q and k: x * rsqrt(mean(x^2) + eps) *
// weight (if weights), then the half-split rotation of the first `rot` dimensions; one rounding. With `v_share`
// s > 1 the row and the page hold kv_heads / s value heads (s key heads read one value head); with `v_from_keys` value
// head g is key head g as projected (bias added, before norm and rotation; there are no value columns then). `pages` null: kv_heads is 0,
// the rows hold queries alone and nothing is stored.
template <typename T>
__global__ void __launch_bounds__(256) head_prepare_kernel(const T* __restrict__ qkv, T* __restrict__ q_out, int heads,
                                                           int kv_heads, int dim, int vdim,
                                                           const T* __restrict__ q_weight, const T* __restrict__ k_weight,
                                                           float eps, const float* __restrict__ table, int rot,
                                                           int table_rows, const int32_t* __restrict__ positions,
                                                           T* __restrict__ pages, const int32_t* __restrict__ write_page,
                                                           const int32_t* __restrict__ write_off, int page_size,
                                                           int num_pages, const float* __restrict__ bias, int64_t stride,
                                                           int v_from_keys, int v_share) {
  const int t = blockIdx.x;
  const int hs = blockIdx.y * 4 + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  const int v_heads = kv_heads / v_share;
  if (hs >= heads + kv_heads + v_heads) return;
  const int64_t page_len = (int64_t)kv_heads * page_size * dim + (int64_t)v_heads * page_size * vdim;
  const T* row = qkv + (int64_t)t * stride;
  const int page = pages ? write_page[t] : -1, off = pages ? write_off[t] : -1;
  const bool page_ok = page >= 0 && page < num_pages && off >= 0 && off < page_size;
  if (hs >= heads + kv_heads) {                       // a value head: stored as it is
    const int hv = hs - heads - kv_heads;
    if (!page_ok) return;
    const int64_t col = v_from_keys ? (int64_t)(heads + hv) * dim : (int64_t)(heads + kv_heads) * dim + (int64_t)hv * vdim;
    const T* src = row + col;
    T* dst = pages + page * page_len + (int64_t)kv_heads * page_size * dim + (int64_t)hv * vdim * page_size + off;
    if (bias) {
      for (int d = lane; d < vdim; d += WAVE)
        dst[(int64_t)d * page_size] = Elem<T>::store(Elem<T>::load(src[d]) + bias[col + d]);
    } else {
      for (int d = lane; d < vdim; d += WAVE) dst[(int64_t)d * page_size] = src[d];
    }
    return;
  }
  const bool is_q = hs < heads;
  if (!is_q && !page_ok) return;
  const T* src = row + (int64_t)hs * dim;
  T* dst = is_q ? q_out + ((int64_t)t * heads + hs) * dim
                : pages + page * page_len + ((int64_t)(hs - heads) * page_size + off) * dim;
  const T* w = is_q ? q_weight : k_weight;
  const float* bs = bias ? bias + (int64_t)hs * dim : nullptr;
  auto in = [&](int d) { return Elem<T>::load(src[d]) + (bs ? bs[d] : 0.f); };
  float r = 1.f;
  if (w) {
    float ss = 0.f;
    for (int d = lane; d < dim; d += WAVE) {
      const float v = in(d);
      ss += v * v;
    }
    r = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
  }
  const int half = rot / 2;
  if (table) {
    int pos = positions[t];
    pos = pos < 0 ? 0 : (pos >= table_rows ? table_rows - 1 : pos);
    const float* cs = table + (int64_t)pos * rot;
    for (int p = lane; p < half; p += WAVE) {
      const float a = in(p) * r * (w ? Elem<T>::load(w[p]) : 1.f);
      const float b = in(p + half) * r * (w ? Elem<T>::load(w[p + half]) : 1.f);
      const float c = cs[p], s = cs[half + p];
      dst[p] = Elem<T>::store(a * c - b * s);
      dst[p + half] = Elem<T>::store(b * c + a * s);
    }
  }
  for (int d = (table ? rot : 0) + lane; d < dim; d += WAVE)
    dst[d] = Elem<T>::store(in(d) * r * (w ? Elem<T>::load(w[d]) : 1.f));
}

// The general kernel (any dtype and sizes; the decode rows of every step): one block of four waves per (token, head).
// The query's keys are walked in tiles of 64 from the oldest visible one; wave w takes tiles w, w + 4, ... A lane takes
// one key of a tile: its score over D (the query comes from LDS) and its weight; then the lanes turn to the value
// columns and add the tile's weighted values, each weight handed round from the lane that holds it. The four waves' sums
// are added in wave order at the end, so the order of every sum is decided by the query's position alone.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256) sigmoid_attention_kernel(const T* __restrict__ q, T* __restrict__ out,
                                                                const T* __restrict__ pages,
                                                                const int32_t* __restrict__ table, int table_stride,
                                                                const int32_t* __restrict__ slots,
                                                                const int32_t* __restrict__ token_row,
                                                                const int32_t* __restrict__ positions,
                                                                const int32_t* __restrict__ query_start,
                                                                const int32_t* __restrict__ row_ids, int heads,
                                                                int kv_heads, int dim, int vdim, int page_size,
                                                                const float* __restrict__ bias, float scale, int window,
                                                                const T* __restrict__ gate) {
  __shared__ float q_s[SIG_MAX_D];
  __shared__ float sum_s[4][SIG_MAX_D];
  const int w = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int t = row_ids ? query_start[row_ids[blockIdx.x]] : blockIdx.x;   // the one token of a listed row, or every token
  const int h = blockIdx.y;
  const int pos = positions[t];
  const int hk = h / (heads / kv_heads);
  const int32_t* trow = table + (int64_t)slots[token_row[t]] * table_stride;
  const int64_t page_len = (int64_t)kv_heads * page_size * (dim + vdim);
  const int64_t val_base = (int64_t)kv_heads * page_size * dim;
  const T* qp = q + ((int64_t)t * heads + h) * dim;
  for (int d = threadIdx.x; d < dim; d += 256) q_s[d] = Elem<T>::load(qp[d]);
  __syncthreads();
  const float head_bias = bias ? bias[h] : 0.f;
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  float acc[SIG_MAX_D / WAVE];
#pragma unroll
  for (int i = 0; i < SIG_MAX_D / WAVE; ++i) acc[i] = 0.f;
  constexpr int V = Elem<T>::kVec;

  for (int j0 = first + w * WAVE; j0 <= pos; j0 += 4 * WAVE) {
    const int key = j0 + lane;
    float p = 0.f;
    int64_t voff = 0;
    if (key <= pos) {
      const int page = trow[key / page_size];
      const int off = key - (key / page_size) * page_size;
      const T* kp = pages + page * page_len + ((int64_t)hk * page_size + off) * dim;
      voff = page * page_len + val_base + (int64_t)hk * vdim * page_size + off;
      float dot = 0.f;
      if (VEC) {
        for (int d = 0; d < dim; d += V) {
          const uint4 raw = *reinterpret_cast<const uint4*>(kp + d);
          const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
          for (int i = 0; i < V; ++i) dot += q_s[d + i] * Elem<T>::load(e[i]);
        }
      } else {
        for (int d = 0; d < dim; ++d) dot += q_s[d] * Elem<T>::load(kp[d]);
      }
      p = 1.0f / (1.0f + expf(-(dot * scale + head_bias)));
    }
    const int count = min(WAVE, pos - j0 + 1);
    for (int j = 0; j < count; ++j) {                 // j is the same in every lane: the holder's values come by readlane
      const float pj = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(p), j));
      const uint32_t lo = __builtin_amdgcn_readlane((uint32_t)(voff & 0xffffffffu), j);
      const uint32_t hi = __builtin_amdgcn_readlane((uint32_t)((uint64_t)voff >> 32), j);
      const T* vp = pages + (int64_t)(((uint64_t)hi << 32) | lo);
#pragma unroll
      for (int i = 0; i < SIG_MAX_D / WAVE; ++i) {
        const int d = lane + i * WAVE;
        if (d < vdim) acc[i] += pj * Elem<T>::load(vp[(int64_t)d * page_size]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < SIG_MAX_D / WAVE; ++i) {
    const int d = lane + i * WAVE;
    if (d < vdim) sum_s[w][d] = acc[i];
  }
  __syncthreads();
  for (int d = threadIdx.x; d < vdim; d += 256) {
    const int64_t at = ((int64_t)t * heads + h) * vdim + d;
    float o = ((sum_s[0][d] + sum_s[1][d]) + sum_s[2][d]) + sum_s[3][d];
    if (gate) o *= 1.0f / (1.0f + expf(-Elem<T>::load(gate[at])));
    out[at] = Elem<T>::store(o);
  }
}
}  // namespace

extern "C" int holon_head_prepare(const void* qkv, void* q_out, int tokens, int heads, int kv_heads, int dim, int vdim,
                                  const void* q_weight, const void* k_weight, float eps, const float* table, int rot,
                                  int table_rows, const int32_t* positions, void* pages, const int32_t* write_page,
                                  const int32_t* write_off, int page_size, int num_pages, int dtype, const float* bias,
                                  int stride, int v_from_keys, int v_share, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && kv_heads >= 0 && dim > 0 && vdim > 0 && v_share >= 1 &&
                  kv_heads % v_share == 0 && (!v_from_keys || (vdim == dim && v_share == 1)),
              "head_prepare: %d/%d heads of %d/%d, a value head for every %d key heads%s", heads, kv_heads, dim, vdim,
              v_share, v_from_keys ? ", values from the keys" : "");
  HOLON_CHECK((table == nullptr && rot == 0) || (rot > 0 && rot % 2 == 0 && rot <= dim && table_rows > 0),
              "head_prepare: %d rotary dimensions for heads of %d", rot, dim);
  HOLON_CHECK((q_weight == nullptr) == (k_weight == nullptr), "head_prepare: one norm weight without the other");
  HOLON_CHECK(pages ? (kv_heads > 0 && page_size > 0 && num_pages > 0 && write_page && write_off) : kv_heads == 0,
              "head_prepare: bad page geometry, or key heads without pages to store them");
  const int64_t width = (int64_t)(heads + kv_heads) * dim + (v_from_keys ? 0 : (int64_t)(kv_heads / v_share) * vdim);
  HOLON_CHECK(stride >= width, "head_prepare: rows of %d values hold no %lld columns", stride, (long long)width);
  if (tokens == 0) return 0;
  HOLON_CHECK((heads + 2 * kv_heads + 3) / 4 <= 65535, "head_prepare: too many heads for one launch");
  const dim3 grid(tokens, (heads + 2 * kv_heads + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    head_prepare_kernel<float><<<grid, 256, 0, s>>>((const float*)qkv, (float*)q_out, heads, kv_heads, dim, vdim,
                                                    (const float*)q_weight, (const float*)k_weight, eps, table, rot,
                                                    table_rows, positions, (float*)pages, write_page, write_off,
                                                    page_size, num_pages, bias, stride, v_from_keys, v_share);
  else
    head_prepare_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)qkv, (bf16_t*)q_out, heads, kv_heads, dim, vdim,
                                                     (const bf16_t*)q_weight, (const bf16_t*)k_weight, eps, table, rot,
                                                     table_rows, positions, (bf16_t*)pages, write_page, write_off,
                                                     page_size, num_pages, bias, stride, v_from_keys, v_share);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_sigmoid_attention(const void* q, void* out, const void* pages, const int32_t* table,
                                       int table_stride, const int32_t* slots, const int32_t* token_row,
                                       const int32_t* positions, const int32_t* query_start, const int32_t* row_ids,
                                       int tokens, int heads, int kv_heads, int dim, int vdim, int page_size,
                                       int num_pages, const float* bias, float scale, int window, const void* gate,
                                       int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "sigmoid_attention: %d/%d heads", heads,
              kv_heads);
  HOLON_CHECK(dim > 0 && dim <= SIG_MAX_D && vdim > 0 && vdim <= SIG_MAX_D,
              "sigmoid_attention: head sizes %d/%d (at most %d)", dim, vdim, SIG_MAX_D);
  HOLON_CHECK(page_size > 0 && num_pages > 0 && window >= 0 && table_stride > 0, "sigmoid_attention: bad page geometry");
  HOLON_CHECK(row_ids == nullptr || query_start != nullptr, "sigmoid_attention: listed rows need query_start");
  if (tokens == 0) return 0;        // (with row_ids: `tokens` is the number of listed rows)
  HOLON_CHECK(heads <= 65535, "sigmoid_attention: %d heads exceed one launch", heads);
  const dim3 grid(tokens, heads);
  hipStream_t s = (hipStream_t)stream;
  const int vec = dtype == HOLON_F32 ? 4 : 8;
  const bool aligned = dim % vec == 0 && ((int64_t)vdim * page_size) % vec == 0 && (uintptr_t)pages % 16 == 0;
#define SIG_LAUNCH(T, VEC)                                                                                            \
  sigmoid_attention_kernel<T, VEC><<<grid, 256, 0, s>>>((const T*)q, (T*)out, (const T*)pages, table, table_stride,  \
                                                        slots, token_row, positions, query_start, row_ids, heads,     \
                                                        kv_heads, dim, vdim, page_size, bias, scale, window,         \
                                                        (const T*)gate)
  if (dtype == HOLON_F32) { if (aligned) SIG_LAUNCH(float, true); else SIG_LAUNCH(float, false); }
  else { if (aligned) SIG_LAUNCH(bf16_t, true); else SIG_LAUNCH(bf16_t, false); }
#undef SIG_LAUNCH
  HOLON_LAUNCH_OK();
  return 0;
}
