// Softmax attention over a paged cache whose keys and values may differ in width, with an optional sliding window and an
// optional sink (one scalar per head whose exponential joins the normaliser; nothing is read from the cache for it). The general kernel: any
// element type, any sizes. Options on the scores: a tanh cap (s <- cap tanh(s / cap)), a distance bias per head
// (s <- s - r1 ln(1 + r2 (i - j)) for query i and key j), and under a window the first tokens of the sequence kept
// visible (key j is seen if j <= i and (i - j < window or j < keep_first)).
//
// A page of one site holds P tokens: keys [Hkv, P, D] (a token's key is a row), then values [Hkv, V, P] (transposed
// inside the page); with `v_share` s > 1 only Hkv / s value heads, key head h reading value head h / s. One block of four waves per (token, head). Keys are walked in tiles of 64 that start at multiples
// of 64 (so a tile is whole pages wherever P divides 64), wave w taking tiles w, w + 4, ... of those the query sees (the
// tiles of the kept first tokens, where they lie wholly before the window's first tile, then the window's); a
// lane takes one key of a tile: its score over D, with the query in LDS. For the values the lanes turn to the value
// columns: column d of a page is P neighbouring values, which a lane reads as 16-byte vectors and weighs with the
// tile's weights, handed round from the lanes that hold them. Every wave keeps a running maximum, sum and weighted
// values; the four are combined at the end in wave order, the sink joining there. Which keys a wave takes and in which
// order is decided by the query's position alone. Scores, weights and sums are float32.
#include "common.h"
#include "holon_hip.h"

#define SMX_MAX_D 1024

namespace {

template <typename T, bool PAGED_VEC>
__global__ void __launch_bounds__(256) softmax_attention_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ pages, const int32_t* __restrict__ table,
    int table_stride, int table_rows, const int32_t* __restrict__ slots, const int32_t* __restrict__ token_row,
    const int32_t* __restrict__ positions, int heads, int kv_heads, int dim, int vdim, int page_size, int num_pages,
    const float* __restrict__ sink, float scale, int window, int key_vec, float softcap,
    const float* __restrict__ r1, const float* __restrict__ r2, int keep_first, int v_share) {
  __shared__ float q_s[SMX_MAX_D];
  __shared__ float sum_s[4][SMX_MAX_D];
  __shared__ float ml_s[4][2];
  const int w = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int t = blockIdx.x, h = blockIdx.y;
  const int pos = positions[t];
  const int hk = h / (heads / kv_heads);
  int slot = slots[token_row[t]];
  slot = slot < 0 ? 0 : (slot >= table_rows ? table_rows - 1 : slot);
  const int32_t* trow = table + (int64_t)slot * table_stride;
  // (v_share key heads read one value head: a page then holds kv_heads / v_share value heads behind its keys)
  const int64_t page_len = (int64_t)kv_heads * page_size * dim + (int64_t)(kv_heads / v_share) * page_size * vdim;
  const int64_t val_base = (int64_t)kv_heads * page_size * dim + (int64_t)(hk / v_share) * vdim * page_size;
  const T* qp = q + ((int64_t)t * heads + h) * dim;
  for (int d = threadIdx.x; d < dim; d += 256) q_s[d] = Elem<T>::load(qp[d]);
  __syncthreads();
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  const int kept = window > 0 && keep_first > 0 ? min(keep_first, first) : 0;      // keys 0 .. kept - 1 are seen too
  const int tile_first = first / WAVE;
  const int extra = min((kept + WAVE - 1) / WAVE, tile_first);     // tiles of kept keys wholly before the window's first
  const int n_tiles = extra + (pos / WAVE - tile_first + 1);
  const float b1 = r1 ? r1[h] : 0.f, b2 = r1 ? r2[h] : 0.f;
  float m = -INFINITY, l = 0.f;
  float acc[SMX_MAX_D / WAVE];
#pragma unroll
  for (int i = 0; i < SMX_MAX_D / WAVE; ++i) acc[i] = 0.f;
  constexpr int VEC = Elem<T>::kVec;     // key_vec: every key row starts on a 16-byte border and is whole vectors

  for (int n = w; n < n_tiles; n += 4) {
    const int j0 = (n < extra ? n : tile_first + n - extra) * WAVE;
    const int key = j0 + lane;
    const bool seen = key <= pos && (key >= first || key < kept);
    float s = -INFINITY;
    int page = -1;
    if (seen && key / page_size < table_stride) {
      page = trow[key / page_size];
      if (page < 0 || page >= num_pages) page = -1;      // a table that does not hold the key: the key is not seen
    }
    if (page >= 0) {
      const int off = key % page_size;
      const T* kp = pages + page * page_len + ((int64_t)hk * page_size + off) * dim;
      float dot = 0.f;
      if (key_vec) {
        for (int d = 0; d < dim; d += VEC) {
          const uint4 raw = *reinterpret_cast<const uint4*>(kp + d);
          const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
          for (int i = 0; i < VEC; ++i) dot += q_s[d + i] * Elem<T>::load(e[i]);
        }
      } else {
        for (int d = 0; d < dim; ++d) dot += q_s[d] * Elem<T>::load(kp[d]);
      }
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      if (r1) s -= b1 * log1pf(b2 * (float)(pos - key));
    }
    const float m_new = fmaxf(m, wave_max(s));
    if (m_new == -INFINITY) continue;                    // nothing seen in this tile (the same in every lane)
    const float alpha = expf(m - m_new);                 // m = -inf before the first key: 0
    const float p = page >= 0 ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < SMX_MAX_D / WAVE; ++i) acc[i] *= alpha;
    if (PAGED_VEC) {
      // the tile is 64 / P whole pages; a lane reads its columns' P values of a page as vectors
      const int per = WAVE / page_size;
      const uint64_t have = __ballot(page >= 0);         // the lanes whose key is seen and held
      for (int g = 0; g < per; ++g) {
        const int k0 = g * page_size;                    // the page's first key among the tile's
        const uint64_t in_page = (have >> k0) & (page_size >= 64 ? ~0ull : ((1ull << page_size) - 1));
        if (!in_page) continue;
        const int pg = __builtin_amdgcn_readlane(page, k0 + __builtin_ctzll(in_page));
        const T* vp = pages + pg * page_len + val_base;
#pragma unroll
        for (int i = 0; i < SMX_MAX_D / WAVE; ++i) {
          const int d = lane + i * WAVE;
          if (d >= vdim) break;
          const T* col = vp + (int64_t)d * page_size;
          float a = acc[i];
          for (int o = 0; o < page_size; o += VEC) {
            const uint4 raw = *reinterpret_cast<const uint4*>(col + o);
            const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
            for (int u = 0; u < VEC; ++u) {
              const float pj = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(p), k0 + o + u));
              a += pj * Elem<T>::load(e[u]);
            }
          }
          acc[i] = a;
        }
      }
    } else {
      const int count = min(WAVE, pos - j0 + 1);
      for (int j = 0; j < count; ++j) {                  // j is the same in every lane
        const int pg = __builtin_amdgcn_readlane(page, j);
        if (pg < 0) continue;
        const float pj = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(p), j));
        const T* vp = pages + pg * page_len + val_base + (j0 + j) % page_size;
#pragma unroll
        for (int i = 0; i < SMX_MAX_D / WAVE; ++i) {
          const int d = lane + i * WAVE;
          if (d < vdim) acc[i] += pj * Elem<T>::load(vp[(int64_t)d * page_size]);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < SMX_MAX_D / WAVE; ++i) {
    const int d = lane + i * WAVE;
    if (d < vdim) sum_s[w][d] = acc[i];
  }
  if (lane == 0) { ml_s[w][0] = m; ml_s[w][1] = l; }
  __syncthreads();
  float top = sink ? sink[h] : -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; ++i) top = fmaxf(top, ml_s[i][0]);
  float f[4], den = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[i] = ml_s[i][0] == -INFINITY ? 0.f : expf(ml_s[i][0] - top);
    den += ml_s[i][1] * f[i];
  }
  if (sink) den += expf(sink[h] - top);
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  for (int d = threadIdx.x; d < vdim; d += 256) {
    const float o = ((sum_s[0][d] * f[0] + sum_s[1][d] * f[1]) + sum_s[2][d] * f[2]) + sum_s[3][d] * f[3];
    out[((int64_t)t * heads + h) * vdim + d] = Elem<T>::store(o * inv);
  }
}
}  // namespace

extern "C" int holon_softmax_attention(const void* q, void* out, const void* pages, const int32_t* table,
                                       int table_stride, int table_rows, const int32_t* slots,
                                       const int32_t* token_row, const int32_t* positions, int tokens, int heads,
                                       int kv_heads, int dim, int vdim, int page_size, int num_pages, const float* sink,
                                       float scale, int window, int dtype, float softcap, const float* r1,
                                       const float* r2, int keep_first, int v_share, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "softmax_attention: %d/%d heads", heads,
              kv_heads);
  HOLON_CHECK(v_share >= 1 && kv_heads % v_share == 0, "softmax_attention: %d key heads do not share value heads by %d",
              kv_heads, v_share);
  HOLON_CHECK(dim > 0 && dim <= SMX_MAX_D && vdim > 0 && vdim <= SMX_MAX_D,
              "softmax_attention: head sizes %d/%d (at most %d)", dim, vdim, SMX_MAX_D);
  HOLON_CHECK(page_size > 0 && num_pages > 0 && window >= 0 && table_stride > 0 && table_rows > 0,
              "softmax_attention: bad page geometry");
  HOLON_CHECK(softcap >= 0.f && keep_first >= 0 && (r1 == nullptr) == (r2 == nullptr),
              "softmax_attention: a cap of %g, %d kept tokens, a distance bias of two numbers a head", softcap, keep_first);
  if (tokens == 0) return 0;
  HOLON_CHECK(heads <= 65535, "softmax_attention: %d heads exceed one launch", heads);
  const dim3 grid(tokens, heads);
  hipStream_t s = (hipStream_t)stream;
  const int vec = dtype == HOLON_F32 ? 4 : 8;
  const bool based = (uintptr_t)pages % 16 == 0;
  const int key_vec = based && dim % vec == 0 && ((int64_t)vdim * page_size) % vec == 0;
  const bool paged_vec = based && WAVE % page_size == 0 && page_size % vec == 0;
#define SMX_LAUNCH(T, PV)                                                                                            \
  softmax_attention_kernel<T, PV><<<grid, 256, 0, s>>>((const T*)q, (T*)out, (const T*)pages, table, table_stride,   \
                                                       table_rows, slots, token_row, positions, heads, kv_heads, dim, \
                                                       vdim, page_size, num_pages, sink, scale, window, key_vec,     \
                                                       softcap, r1, r2, keep_first, v_share)
  if (dtype == HOLON_F32) { if (paged_vec) SMX_LAUNCH(float, true); else SMX_LAUNCH(float, false); }
  else { if (paged_vec) SMX_LAUNCH(bf16_t, true); else SMX_LAUNCH(bf16_t, false); }
#undef SMX_LAUNCH
  HOLON_LAUNCH_OK();
  return 0;
}

// -- the latent attention's small steps ---------------------------------------------------------------------------------
namespace {

// One block a token. `both` [T, q_rank + kv_rank] holds the two latents' projections side by side. Each is divided by
// its root mean square (eps inside the root) and multiplied by its weight, float32 inside, one rounding: the first goes
// to `cq` [T, q_rank]; the second is the token's entry in the cache, stored twice in the page it belongs to, as a key
// (a row of [P, kv_rank]) and as a value (a column of [kv_rank, P]).
template <typename T>
__global__ void __launch_bounds__(256) latent_prepare_kernel(const T* __restrict__ both, int q_rank, int kv_rank,
                                                             const T* __restrict__ q_weight, const T* __restrict__ c_weight,
                                                             float eps, T* __restrict__ cq, T* __restrict__ pages,
                                                             const int32_t* __restrict__ write_page,
                                                             const int32_t* __restrict__ write_off, int page_size,
                                                             int num_pages) {
  __shared__ float part[2][4];
  const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* row = both + (int64_t)t * (q_rank + kv_rank);
  float sq = 0.f, sc = 0.f;
  for (int d = threadIdx.x; d < q_rank; d += 256) { const float v = Elem<T>::load(row[d]); sq += v * v; }
  for (int d = threadIdx.x; d < kv_rank; d += 256) { const float v = Elem<T>::load(row[q_rank + d]); sc += v * v; }
  sq = wave_sum(sq);
  sc = wave_sum(sc);
  if (lane == 0) { part[0][wave] = sq; part[1][wave] = sc; }
  __syncthreads();
  const float rq = 1.0f / sqrtf(((part[0][0] + part[0][1]) + (part[0][2] + part[0][3])) / (float)q_rank + eps);
  const float rc = 1.0f / sqrtf(((part[1][0] + part[1][1]) + (part[1][2] + part[1][3])) / (float)kv_rank + eps);
  for (int d = threadIdx.x; d < q_rank; d += 256)
    cq[(int64_t)t * q_rank + d] = Elem<T>::store(Elem<T>::load(row[d]) * rq * Elem<T>::load(q_weight[d]));
  const int page = write_page[t], off = write_off[t];
  if (page < 0 || page >= num_pages || off < 0 || off >= page_size) return;
  T* keys = pages + (int64_t)page * 2 * page_size * kv_rank;
  T* vals = keys + (int64_t)page_size * kv_rank;
  for (int d = threadIdx.x; d < kv_rank; d += 256) {
    const T c = Elem<T>::store(Elem<T>::load(row[q_rank + d]) * rc * Elem<T>::load(c_weight[d]));
    keys[(int64_t)off * kv_rank + d] = c;
    vals[(int64_t)d * page_size + off] = c;
  }
}

// y[t, h, b] = sum_a x[t, h, a] w[h, b, a] for steps of few rows: a block takes a head and 16 of its output columns,
// the rows' values of that head wait in LDS, and sixteen lanes share a column (each a sixteenth of A, in the order of
// the lane), added up in a fixed order. float32 sums, one rounding.
template <typename T>
__global__ void __launch_bounds__(256) head_linear_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                          T* __restrict__ y, int rows, int heads, int A, int B,
                                                          int y_head) {      // y_head: values between two heads of y
  extern __shared__ float xs[];                          // [rows, A]
  const int h = blockIdx.x, b = blockIdx.y * 16 + threadIdx.x / 16, part = threadIdx.x % 16;
  for (int i = threadIdx.x; i < rows * A; i += 256) {
    const int t = i / A, a = i - t * A;
    xs[i] = Elem<T>::load(x[((int64_t)t * heads + h) * A + a]);
  }
  __syncthreads();
  const T* wr = w + ((int64_t)h * B + (b < B ? b : 0)) * A;
  constexpr int VEC = Elem<T>::kVec;
  const bool wide = A % (16 * VEC) == 0 && (uintptr_t)w % 16 == 0;      // a lane's share as 16-byte loads
  for (int t0 = 0; t0 < rows; t0 += 8) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (wide) {
      for (int a = part * VEC; a < A; a += 16 * VEC) {
        const uint4 raw = *reinterpret_cast<const uint4*>(wr + a);
        const T* e = reinterpret_cast<const T*>(&raw);
        float wv[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) wv[i] = Elem<T>::load(e[i]);
#pragma unroll
        for (int r = 0; r < 8; ++r)
          if (t0 + r < rows) {
            const float* xr = xs + (t0 + r) * A + a;
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[r] += xr[i] * wv[i];
          }
      }
    } else {
      for (int a = part; a < A; a += 16) {
        const float wv = Elem<T>::load(wr[a]);
#pragma unroll
        for (int r = 0; r < 8; ++r)
          if (t0 + r < rows) acc[r] += xs[(t0 + r) * A + a] * wv;
      }
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      float v = acc[r];
      v += __shfl_xor(v, 1, WAVE);
      v += __shfl_xor(v, 2, WAVE);
      v += __shfl_xor(v, 4, WAVE);
      v += __shfl_xor(v, 8, WAVE);
      if (part == 0 && b < B && t0 + r < rows) y[((int64_t)(t0 + r) * heads + h) * y_head + b] = Elem<T>::store(v);
    }
  }
}
}  // namespace

extern "C" int holon_latent_prepare(const void* both, int tokens, int q_rank, int kv_rank, const void* q_weight,
                                    const void* c_weight, float eps, void* cq, void* pages, const int32_t* write_page,
                                    const int32_t* write_off, int page_size, int num_pages, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && q_rank > 0 && kv_rank > 0 && page_size > 0 && num_pages > 0,
              "latent_prepare: latents of %d and %d, pages of %d", q_rank, kv_rank, page_size);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    latent_prepare_kernel<float><<<tokens, 256, 0, s>>>((const float*)both, q_rank, kv_rank, (const float*)q_weight,
                                                       (const float*)c_weight, eps, (float*)cq, (float*)pages,
                                                       write_page, write_off, page_size, num_pages);
  else
    latent_prepare_kernel<bf16_t><<<tokens, 256, 0, s>>>((const bf16_t*)both, q_rank, kv_rank, (const bf16_t*)q_weight,
                                                        (const bf16_t*)c_weight, eps, (bf16_t*)cq, (bf16_t*)pages,
                                                        write_page, write_off, page_size, num_pages);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_head_linear_rows(const void* x, const void* w, void* y, int rows, int heads, int A, int B,
                                      int y_head, int dtype, void* stream) {
  HOLON_CHECK(rows >= 1 && rows <= 16 && heads > 0 && heads <= 65535 && A > 0 && B > 0 && y_head >= B &&
                  (int64_t)rows * A * 4 <= 48 * 1024,
              "head_linear (few rows): %d rows, %d heads of %d -> %d (in steps of %d)", rows, heads, A, B, y_head);
  const dim3 grid(heads, (B + 15) / 16);
  const size_t lds = (size_t)rows * A * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    head_linear_kernel<float><<<grid, 256, lds, s>>>((const float*)x, (const float*)w, (float*)y, rows, heads, A, B, y_head);
  else
    head_linear_kernel<bf16_t><<<grid, 256, lds, s>>>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, rows, heads, A, B, y_head);
  HOLON_LAUNCH_OK();
  return 0;
}

// -- preparing the merged projections of the two attention mixers -------------------------------------------------------
namespace {

// Sum over a block of 256 threads of two values at once; waves are added in order.
__device__ __forceinline__ void block_sum2_256(float& a, float& b, float (*part)[4]) {
  a = wave_sum(a);
  b = wave_sum(b);
  __syncthreads();
  if (threadIdx.x % WAVE == 0) { part[0][threadIdx.x / WAVE] = a; part[1][threadIdx.x / WAVE] = b; }
  __syncthreads();
  a = (part[0][0] + part[0][1]) + (part[0][2] + part[0][3]);
  b = (part[1][0] + part[1][1]) + (part[1][2] + part[1][3]);
}

// One block a token. `qkv` [T, H D + G D + G V]: all of the token's query values are divided by their root mean square
// as one vector and multiplied by q_weight [H D], all of its key values likewise with k_weight [G D] (eps inside the
// root, float32 inside, one rounding). Queries go to `q` [T, H, D]; keys and values into the token's page: keys
// [G, P, D], then values [G, V, P].
template <typename T>
__global__ void __launch_bounds__(256) whole_norm_prepare_kernel(
    const T* __restrict__ qkv, int heads, int kv_heads, int dim, int vdim, const T* __restrict__ q_weight,
    const T* __restrict__ k_weight, float eps, T* __restrict__ q, T* __restrict__ pages,
    const int32_t* __restrict__ write_page, const int32_t* __restrict__ write_off, int page_size, int num_pages) {
  __shared__ float part[2][4];
  const int t = blockIdx.x;
  const int nq = heads * dim, nk = kv_heads * dim, nv = kv_heads * vdim;
  const T* row = qkv + (int64_t)t * (nq + nk + nv);
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < nq; c += 256) { const float v = Elem<T>::load(row[c]); sq += v * v; }
  for (int c = threadIdx.x; c < nk; c += 256) { const float v = Elem<T>::load(row[nq + c]); sk += v * v; }
  block_sum2_256(sq, sk, part);
  const float rq = 1.0f / sqrtf(sq / (float)nq + eps), rk = 1.0f / sqrtf(sk / (float)nk + eps);
  for (int c = threadIdx.x; c < nq; c += 256)
    q[(int64_t)t * nq + c] = Elem<T>::store(Elem<T>::load(row[c]) * rq * Elem<T>::load(q_weight[c]));
  const int page = write_page[t], off = write_off[t];
  if (page < 0 || page >= num_pages || off < 0 || off >= page_size) return;
  T* keys = pages + (int64_t)page * kv_heads * page_size * (dim + vdim);
  T* vals = keys + (int64_t)kv_heads * page_size * dim;
  for (int c = threadIdx.x; c < nk; c += 256) {
    const int g = c / dim, d = c - g * dim;
    keys[((int64_t)g * page_size + off) * dim + d] =
        Elem<T>::store(Elem<T>::load(row[nq + c]) * rk * Elem<T>::load(k_weight[c]));
  }
  for (int c = threadIdx.x; c < nv; c += 256) vals[(int64_t)c * page_size + off] = row[nq + nk + c];
}

// One block a token. `both` [T, H (dim + rot) + kv_rank + rot]: every head's query as [dim unrotated, rot rotated], then
// the latent's projection and one rotated key part. The latent is RMS-normed with c_weight; the first `rd` of the `rot`
// dimensions of every rotated part turn by the token's position (pairs (i, i + rd / 2), `table` row = rd / 2 cosines,
// then rd / 2 sines). Unrotated query parts go to `qn` [T, H, dim], rotated ones into the last `rot` columns of `full`
// [T, H, kv_rank + rot]; the cache entry [latent, rotated key part] into the token's page as a key row of [P, width]
// and as a value column of [width, P].
template <typename T>
__global__ void __launch_bounds__(256) latent_rope_prepare_kernel(
    const T* __restrict__ both, int heads, int dim, int rot, int kv_rank, const T* __restrict__ c_weight, float eps,
    const float* __restrict__ table, int rd, int table_rows, const int32_t* __restrict__ positions, T* __restrict__ qn,
    T* __restrict__ full, T* __restrict__ pages, const int32_t* __restrict__ write_page,
    const int32_t* __restrict__ write_off, int page_size, int num_pages) {
  __shared__ float part[2][4];
  const int t = blockIdx.x;
  const int per = dim + rot, width = kv_rank + rot, half = rd / 2;
  const T* row = both + (int64_t)t * (heads * per + width);
  const T* tail = row + heads * per;
  float sc = 0.f, unused = 0.f;
  for (int d = threadIdx.x; d < kv_rank; d += 256) { const float v = Elem<T>::load(tail[d]); sc += v * v; }
  block_sum2_256(sc, unused, part);
  const float rc = 1.0f / sqrtf(sc / (float)kv_rank + eps);
  int pos = positions[t];
  pos = pos < 0 ? 0 : (pos >= table_rows && table_rows > 0 ? table_rows - 1 : pos);
  const float* cs = table ? table + (int64_t)pos * rd : nullptr;
  // value r of a rotated part `x` [rot] after the turn
  auto turned = [&](const T* x, int r) -> float {
    const float v = Elem<T>::load(x[r]);
    if (r >= rd || !cs) return v;
    if (r < half) return v * cs[r] - Elem<T>::load(x[r + half]) * cs[half + r];
    return v * cs[r - half] + Elem<T>::load(x[r - half]) * cs[r];
  };
  for (int c = threadIdx.x; c < heads * dim; c += 256) {
    const int h = c / dim, d = c - h * dim;
    qn[(int64_t)t * heads * dim + c] = row[h * per + d];
  }
  for (int c = threadIdx.x; c < heads * rot; c += 256) {
    const int h = c / rot, r = c - h * rot;
    full[((int64_t)t * heads + h) * width + kv_rank + r] = Elem<T>::store(turned(row + h * per + dim, r));
  }
  const int page = write_page[t], off = write_off[t];
  if (page < 0 || page >= num_pages || off < 0 || off >= page_size) return;
  T* keys = pages + (int64_t)page * 2 * page_size * width;
  T* vals = keys + (int64_t)page_size * width;
  for (int d = threadIdx.x; d < width; d += 256) {
    const T e = d < kv_rank ? Elem<T>::store(Elem<T>::load(tail[d]) * rc * Elem<T>::load(c_weight[d]))
                            : Elem<T>::store(turned(tail + kv_rank, d - kv_rank));
    keys[(int64_t)off * width + d] = e;
    vals[(int64_t)d * page_size + off] = e;
  }
}
// x[t, h, :] *= sigmoid(gates[t, h]): one wave a (token, head); the gates are columns of rows `gate_stride` apart.
template <typename T>
__global__ void __launch_bounds__(256) head_gate_kernel(T* __restrict__ x, const T* __restrict__ gates,
                                                        int64_t gate_stride, int64_t pairs, int heads, int vdim) {
  const int64_t at = (int64_t)blockIdx.x * 4 + threadIdx.x / WAVE;
  if (at >= pairs) return;
  const int lane = threadIdx.x % WAVE;
  const int64_t t = at / heads;
  const int h = (int)(at % heads);
  const float g = 1.0f / (1.0f + expf(-Elem<T>::load(gates[t * gate_stride + h])));
  T* row = x + at * vdim;
  for (int d = lane; d < vdim; d += WAVE) row[d] = Elem<T>::store(Elem<T>::load(row[d]) * g);
}

// x[t, :] += bias: the sum in float32, one rounding.
template <typename T>
__global__ void __launch_bounds__(256) add_bias_kernel(T* __restrict__ x, const float* __restrict__ bias, int dim) {
  T* row = x + (int64_t)blockIdx.x * dim;
  for (int d = threadIdx.x; d < dim; d += 256) row[d] = Elem<T>::store(Elem<T>::load(row[d]) + bias[d]);
}

// Two maps' results to one: y [T, G, 2, R, V] (kv head, map, head within the group) -> out [T, G, R, V]:
// u = y1 - lam y2, u / sqrt(mean(u^2) + eps) * gain over a head's V values. One wave a (token, head).
template <typename T>
__global__ void __launch_bounds__(256) diff_combine_kernel(const T* __restrict__ y, T* __restrict__ out, int64_t pairs,
                                                           int heads, int group, int vdim, float lam, float eps,
                                                           float gain) {
  const int64_t at = (int64_t)blockIdx.x * 4 + threadIdx.x / WAVE;
  if (at >= pairs) return;
  const int lane = threadIdx.x % WAVE;
  const int64_t t = at / heads;
  const int h = (int)(at % heads), g = h / group, j = h % group;
  const T* first = y + ((t * 2 * heads) + (int64_t)(g * 2) * group + j) * vdim;
  const T* second = first + (int64_t)group * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += WAVE) {
    const float u = Elem<T>::load(first[d]) - lam * Elem<T>::load(second[d]);
    ss += u * u;
  }
  const float r = gain / sqrtf(wave_sum(ss) / (float)vdim + eps);
  T* dst = out + at * vdim;
  for (int d = lane; d < vdim; d += WAVE)
    dst[d] = Elem<T>::store((Elem<T>::load(first[d]) - lam * Elem<T>::load(second[d])) * r);
}
}  // namespace

extern "C" int holon_whole_norm_prepare(const void* qkv, int tokens, int heads, int kv_heads, int dim, int vdim,
                                        const void* q_weight, const void* k_weight, float eps, void* q, void* pages,
                                        const int32_t* write_page, const int32_t* write_off, int page_size,
                                        int num_pages, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0 && page_size > 0 && num_pages > 0,
              "whole_norm_prepare: %d/%d heads of %d/%d, pages of %d", heads, kv_heads, dim, vdim, page_size);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    whole_norm_prepare_kernel<float><<<tokens, 256, 0, s>>>((const float*)qkv, heads, kv_heads, dim, vdim,
                                                           (const float*)q_weight, (const float*)k_weight, eps,
                                                           (float*)q, (float*)pages, write_page, write_off, page_size,
                                                           num_pages);
  else
    whole_norm_prepare_kernel<bf16_t><<<tokens, 256, 0, s>>>((const bf16_t*)qkv, heads, kv_heads, dim, vdim,
                                                            (const bf16_t*)q_weight, (const bf16_t*)k_weight, eps,
                                                            (bf16_t*)q, (bf16_t*)pages, write_page, write_off,
                                                            page_size, num_pages);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_latent_rope_prepare(const void* both, int tokens, int heads, int dim, int rot, int kv_rank,
                                         const void* c_weight, float eps, const float* table, int rd, int table_rows,
                                         const int32_t* positions, void* qn, void* full, void* pages,
                                         const int32_t* write_page, const int32_t* write_off, int page_size,
                                         int num_pages, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && dim > 0 && rot >= 0 && kv_rank > 0 && page_size > 0 && num_pages > 0,
              "latent_rope_prepare: %d heads of %d + %d, a latent of %d, pages of %d", heads, dim, rot, kv_rank, page_size);
  HOLON_CHECK(rd >= 0 && rd % 2 == 0 && rd <= rot && (rd == 0 || (table != nullptr && table_rows > 0)),
              "latent_rope_prepare: %d of %d dimensions rotated, a table of %d rows", rd, rot, table_rows);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    latent_rope_prepare_kernel<float><<<tokens, 256, 0, s>>>((const float*)both, heads, dim, rot, kv_rank,
                                                            (const float*)c_weight, eps, table, rd, table_rows, positions,
                                                            (float*)qn, (float*)full, (float*)pages, write_page,
                                                            write_off, page_size, num_pages);
  else
    latent_rope_prepare_kernel<bf16_t><<<tokens, 256, 0, s>>>((const bf16_t*)both, heads, dim, rot, kv_rank,
                                                             (const bf16_t*)c_weight, eps, table, rd, table_rows,
                                                             positions, (bf16_t*)qn, (bf16_t*)full, (bf16_t*)pages,
                                                             write_page, write_off, page_size, num_pages);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_head_gate(void* x, const void* gates, int64_t gate_stride, int64_t tokens, int heads, int vdim,
                               int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && vdim > 0 && gate_stride >= heads && tokens * heads <= 4LL * 0x7fffffff,
              "head_gate: %lld tokens, %d heads of %d, gates %lld apart", (long long)tokens, heads, vdim,
              (long long)gate_stride);
  if (tokens == 0) return 0;
  const int64_t pairs = tokens * heads;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    head_gate_kernel<float><<<(unsigned)((pairs + 3) / 4), 256, 0, s>>>((float*)x, (const float*)gates, gate_stride,
                                                                        pairs, heads, vdim);
  else
    head_gate_kernel<bf16_t><<<(unsigned)((pairs + 3) / 4), 256, 0, s>>>((bf16_t*)x, (const bf16_t*)gates, gate_stride,
                                                                         pairs, heads, vdim);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_add_bias(void* x, const float* bias, int64_t rows, int dim, int dtype, void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 0x7fffffffLL && dim > 0, "add_bias: rows=%lld dim=%d", (long long)rows, dim);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32) add_bias_kernel<float><<<(unsigned)rows, 256, 0, s>>>((float*)x, bias, dim);
  else add_bias_kernel<bf16_t><<<(unsigned)rows, 256, 0, s>>>((bf16_t*)x, bias, dim);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_diff_combine(const void* y, void* out, int64_t tokens, int heads, int kv_heads, int vdim, float lam,
                                  float eps, float gain, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && vdim > 0 &&
                  tokens * heads <= 4LL * 0x7fffffff,
              "diff_combine: %lld tokens, %d/%d heads of %d", (long long)tokens, heads, kv_heads, vdim);
  if (tokens == 0) return 0;
  const int64_t pairs = tokens * heads;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    diff_combine_kernel<float><<<(unsigned)((pairs + 3) / 4), 256, 0, s>>>((const float*)y, (float*)out, pairs, heads,
                                                                           heads / kv_heads, vdim, lam, eps, gain);
  else
    diff_combine_kernel<bf16_t><<<(unsigned)((pairs + 3) / 4), 256, 0, s>>>((const bf16_t*)y, (bf16_t*)out, pairs, heads,
                                                                            heads / kv_heads, vdim, lam, eps, gain);
  HOLON_LAUNCH_OK();
  return 0;
}
