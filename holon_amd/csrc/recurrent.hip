// Recurrent mixers: a short causal filter with carried inputs, the gated delta rule, a decayed key-value memory with
// token shift, and the small float32 steps around them. A step's rows are ranges of its flat tokens
// (query_start[b] .. query_start[b + 1]), each continuing the state in its request's slot; a row that starts at
// position 0 starts from zeros whatever the slot holds.
//
// The two scans keep a head's matrix S [D, V] in registers through a row's tokens. Its columns never meet, so a wave
// owns 8 of them, eight lanes a column with an eighth of the key rows each; what a token needs of a whole column (a dot
// product with the key, the read-out) is summed over a lane's rows in ascending order and then over the eight lanes in a
// fixed order. Each token's key and query reach the lanes through LDS. The key size is padded to the next instantiated
// one with zeros (a zero key writes nothing).
#include "common.h"
#include "holon_hip.h"

namespace {

template <typename T>
__global__ void causal_conv_kernel(const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ state,
                                   T* __restrict__ y, const int32_t* __restrict__ slots,
                                   const int32_t* __restrict__ starts, const int32_t* __restrict__ query_start,
                                   const int32_t* __restrict__ token_row, int channels, int taps, int add_input,
                                   int act, int keep) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int t = blockIdx.y;
  if (c >= channels) return;
  const int b = keep ? t : token_row[t];               // keep: every row has one token, token t is row t
  const int q0 = keep ? t : query_start[b];
  const int i = t - q0;
  const bool carried = starts[b] > 0;
  T* held = state + (int64_t)slots[b] * (taps - 1) * channels;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int l = i - (taps - 1) + j;
    float v = 0.f;
    if (l >= 0) v = Elem<T>::load(x[(int64_t)(q0 + l) * channels + c]);
    else if (carried) v = Elem<T>::load(held[(int64_t)(taps - 1 + l) * channels + c]);
    acc += Elem<T>::load(w[(int64_t)c * taps + j]) * v;
  }
  if (add_input) acc += Elem<T>::load(x[(int64_t)t * channels + c]);
  if (act) acc = silu<T>(acc);
  y[(int64_t)t * channels + c] = Elem<T>::store(acc);
  if (keep) {                  // the row's one token: this thread alone reads and writes its channel of the slot
    for (int e = 0; e + 2 < taps; ++e)
      held[(int64_t)e * channels + c] = carried ? held[(int64_t)(e + 1) * channels + c] : Elem<T>::store(0.f);
    if (taps > 1) held[(int64_t)(taps - 2) * channels + c] = x[(int64_t)t * channels + c];
  }
}

// The same for prompt portions with a thread taking 16 bytes of channels at a time (channels a multiple of that; rows
// of x, y and the slots then start on 16-byte borders): the same products in the same order.
template <typename T>
__global__ void __launch_bounds__(256) causal_conv_wide_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                               const T* __restrict__ state, T* __restrict__ y,
                                                               const int32_t* __restrict__ slots,
                                                               const int32_t* __restrict__ starts,
                                                               const int32_t* __restrict__ query_start,
                                                               const int32_t* __restrict__ token_row, int channels,
                                                               int taps, int add_input, int act) {
  constexpr int N = Elem<T>::kVec;
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * N;
  const int t = blockIdx.y;
  if (c >= channels) return;
  const int b = token_row[t];
  const int q0 = query_start[b];
  const int i = t - q0;
  const bool carried = starts[b] > 0;
  const T* held = state + (int64_t)slots[b] * (taps - 1) * channels;
  float acc[N];
#pragma unroll
  for (int u = 0; u < N; ++u) acc[u] = 0.f;
  uint4 last = make_uint4(0u, 0u, 0u, 0u);
  for (int j = 0; j < taps; ++j) {
    const int l = i - (taps - 1) + j;
    uint4 raw = make_uint4(0u, 0u, 0u, 0u);
    if (l >= 0) raw = *reinterpret_cast<const uint4*>(x + (int64_t)(q0 + l) * channels + c);
    else if (carried) raw = *reinterpret_cast<const uint4*>(held + (int64_t)(taps - 1 + l) * channels + c);
    const T* v = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int u = 0; u < N; ++u) acc[u] += Elem<T>::load(w[(int64_t)(c + u) * taps + j]) * Elem<T>::load(v[u]);
    last = raw;
  }
  const T* own = reinterpret_cast<const T*>(&last);      // the last tap's input is the token itself
  uint4 out;
  T* o = reinterpret_cast<T*>(&out);
#pragma unroll
  for (int u = 0; u < N; ++u) {
    float a = acc[u];
    if (add_input) a += Elem<T>::load(own[u]);
    if (act) a = silu<T>(a);
    o[u] = Elem<T>::store(a);
  }
  *reinterpret_cast<uint4*>(y + (int64_t)t * channels + c) = out;
}

// After the filter has read the old inputs: the slot takes the row's last taps - 1 inputs, oldest first. A thread
// moves its channel's entries in ascending order and reads only entries at or behind the one it writes.
template <typename T>
__global__ void causal_conv_keep_kernel(const T* __restrict__ x, T* __restrict__ state, const int32_t* __restrict__ slots,
                                        const int32_t* __restrict__ starts, const int32_t* __restrict__ query_start,
                                        int channels, int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int b = blockIdx.y;
  if (c >= channels) return;
  const int q0 = query_start[b], n = query_start[b + 1] - q0;
  const bool carried = starts[b] > 0;
  T* held = state + (int64_t)slots[b] * (taps - 1) * channels;
  for (int i = 0; i < taps - 1; ++i) {
    const int l = n - (taps - 1) + i;
    T v = Elem<T>::store(0.f);
    if (l >= 0) v = x[(int64_t)(q0 + l) * channels + c];
    else if (carried) v = held[(int64_t)(i + n) * channels + c];
    held[(int64_t)i * channels + c] = v;
  }
}

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// One block a token. Waves take the 2 G heads of q and k in turn: unit vectors (q also times D^-0.5); then the step
// sizes and decays of the H heads.
template <typename T>
__global__ void __launch_bounds__(256) delta_prepare_kernel(const T* __restrict__ qkv, const T* __restrict__ ab,
                                                            const float* __restrict__ a_log,
                                                            const float* __restrict__ dt_bias, float* __restrict__ qn,
                                                            float* __restrict__ kn, float* __restrict__ beta,
                                                            float* __restrict__ g, int heads, int kv_heads, int dim,
                                                            int vdim) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int width = 2 * kv_heads * dim + heads * vdim;
  const T* row = qkv + (int64_t)t * width;
  for (int idx = wave; idx < 2 * kv_heads; idx += 4) {
    const bool is_q = idx < kv_heads;
    const int h = is_q ? idx : idx - kv_heads;
    const T* src = row + (int64_t)idx * dim;
    float ss = 0.f;
    for (int d = lane; d < dim; d += WAVE) {
      const float v = Elem<T>::load(src[d]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = (1.0f / sqrtf(ss + 1e-6f)) * (is_q ? 1.0f / sqrtf((float)dim) : 1.0f);
    float* dst = (is_q ? qn : kn) + ((int64_t)t * kv_heads + h) * dim;
    for (int d = lane; d < dim; d += WAVE) dst[d] = Elem<T>::load(src[d]) * r;
  }
  for (int h = threadIdx.x; h < heads; h += 256) {
    const float a = Elem<T>::load(ab[(int64_t)t * 2 * heads + h]);
    const float b = Elem<T>::load(ab[(int64_t)t * 2 * heads + heads + h]);
    beta[(int64_t)t * heads + h] = 1.0f / (1.0f + expf(-b));
    g[(int64_t)t * heads + h] = expf(-expf(a_log[h]) * softplus_f(a + dt_bias[h]));
  }
}

// Sum over the eight adjacent lanes that share a column, by data-parallel moves inside the vector unit (no trip through
// LDS): lane ^ 1, lane ^ 2, then the mirror image inside the eight, which lies in the other four. A fixed order.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float part_sum(float v) {
  v += dpp_move<0xB1>(v);        // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);        // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x141>(v);       // row_half_mirror
  return v;
}

constexpr int SCAN_PARTS = 8;      // lanes a value column is spread over, each with an eighth of the key rows
constexpr int SCAN_COLS = WAVE / SCAN_PARTS;      // value columns a wave owns

// Tokens a wave stages at a time: their operands travel from memory to LDS as one batch of loads while the batch before
// is worked through, so that a token's arithmetic never waits for memory (one token at a time, a step took as long as
// a load: 0.9 us). About a thousand values per operand and batch.
// ARRAYS: operands of D values a token that the scan stages (they decide the block's LDS, and with it how many waves a
// compute unit holds: the scans wait on latencies, so more waves are more throughput).
template <int KD, int ARRAYS> struct ScanChunk {
  static constexpr int kTokens = ARRAYS <= 2 ? (KD <= 64 ? 16 : KD <= 128 ? 8 : 4) : (KD <= 64 ? 8 : KD <= 128 ? 4 : 2);
};

// A long row's tokens in pieces that run side by side, for the delta rule. A token's step is linear in S,
// S <- g (I - beta k k^T) S + beta k v^T, with a matrix in front that does not depend on S. Every piece but a row's last
// first runs on D + V columns: V from zero with the true values (what the piece adds, B) and D from the identity with
// values of zero (the product of its matrices, A); `ab` [pieces, H, D, V + D] takes both. A small kernel walks a row's
// pieces in order, S <- A S + B, leaving each piece's true starting state in `sin` [pieces, H, D, V]; then every piece
// runs again from there and writes its outputs.
struct DeltaPieces {
  int tokens;                  // tokens a piece (0: rows are not cut)
  int mode;                    // 1: B and A of every piece but the last; 2: from the true start, outputs
  const int32_t* base;         // [rows]: the number of row b's first piece among all pieces of the step
  float* ab;
  float* sin;
};

// Per (row, head): S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q. Lane 8 c + p owns rows
// p KD/8 .. (p + 1) KD/8 - 1 of column c of S.
template <int KD, typename T>
__global__ void __launch_bounds__(WAVE) delta_scan_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                                                          const T* __restrict__ qkv, int qkv_stride, int v_offset,
                                                          const float* __restrict__ beta, const float* __restrict__ g,
                                                          float* __restrict__ state, float* __restrict__ out,
                                                          const int32_t* __restrict__ slots,
                                                          const int32_t* __restrict__ starts,
                                                          const int32_t* __restrict__ query_start, int heads,
                                                          int kv_heads, int dim, int vdim, DeltaPieces pc) {
  constexpr int KQ = KD / SCAN_PARTS, TC = ScanChunk<KD, 2>::kTokens, N = TC * KD, PER = (N + WAVE - 1) / WAVE;
  constexpr int VPER = (TC * SCAN_COLS + WAVE - 1) / WAVE;
  __shared__ __attribute__((aligned(16))) float ks[2][N], qs[2][N];
  __shared__ float vs[2][TC * SCAN_COLS], gs[2][TC], bs[2][TC];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const bool local = pc.tokens > 0 && pc.mode == 1;
  const int columns = local ? vdim + dim : vdim;          // the first pass also carries the identity's D columns
  const int col_blocks = (columns + SCAN_COLS - 1) / SCAN_COLS;
  const int piece = blockIdx.z / col_blocks, col_block = blockIdx.z % col_blocks;
  const int part = lane % SCAN_PARTS, col = lane / SCAN_PARTS, j = col_block * SCAN_COLS + col;
  const int hk = h / (heads / kv_heads);
  const bool active = j < columns;
  int lo = query_start[b], hi = query_start[b + 1];
  bool from_slot = true, to_slot = true;
  int64_t piece_no = 0;
  if (pc.tokens > 0) {                                   // (everything here is the same in all of the block's lanes)
    const int pieces = (hi - lo + pc.tokens - 1) / pc.tokens;
    if (piece >= pieces || (local && piece == pieces - 1)) return;
    lo += piece * pc.tokens;
    hi = min(hi, lo + pc.tokens);
    from_slot = piece == 0;
    to_slot = pc.mode == 2 && piece == pieces - 1;
    piece_no = pc.base[b] + piece;
  }
  float* held = state + ((int64_t)slots[b] * heads + h) * dim * vdim;
  const bool carried = starts[b] > 0;
  float S[KQ];
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int row = part * KQ + i;
    const bool in = active && row < dim;
    if (local) S[i] = (in && j >= vdim && row == j - vdim) ? 1.f : 0.f;
    else if (from_slot) S[i] = (carried && in) ? held[(int64_t)row * vdim + j] : 0.f;
    else S[i] = in ? pc.sin[((piece_no - 1) * heads + h) * dim * vdim + (int64_t)row * vdim + j] : 0.f;
  }
  float nk[PER], nq[PER], nv[VPER], ng = 1.f, nb = 0.f;
  auto ask = [&](int t0) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = lane + e * WAVE, tt = idx / KD, i = idx - tt * KD;
      const bool ok = idx < N && t0 + tt < hi && i < dim;
      const int64_t at = ((int64_t)(t0 + tt) * kv_heads + hk) * dim + i;
      nk[e] = ok ? kn[at] : 0.f;
      nq[e] = ok ? qn[at] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < VPER; ++e) {
      const int idx = lane + e * WAVE, tt = idx / SCAN_COLS, jj = col_block * SCAN_COLS + idx % SCAN_COLS;
      const bool ok = idx < TC * SCAN_COLS && t0 + tt < hi && jj < vdim;      // (the identity's columns take v = 0)
      nv[e] = ok ? Elem<T>::load(qkv[(int64_t)(t0 + tt) * qkv_stride + v_offset + h * vdim + jj]) : 0.f;
    }
    const bool ok = lane < TC && t0 + lane < hi;
    ng = ok ? g[(int64_t)(t0 + lane) * heads + h] : 1.f;
    nb = ok ? beta[(int64_t)(t0 + lane) * heads + h] : 0.f;
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = lane + e * WAVE;
      if (idx < N) { ks[buf][idx] = nk[e]; qs[buf][idx] = nq[e]; }
    }
#pragma unroll
    for (int e = 0; e < VPER; ++e) {
      const int idx = lane + e * WAVE;
      if (idx < TC * SCAN_COLS) vs[buf][idx] = nv[e];
    }
    if (lane < TC) { gs[buf][lane] = ng; bs[buf][lane] = nb; }
  };
  if (lo < hi) {
    ask(lo);
    put(0);
  }
  __syncthreads();
  for (int t0 = lo, buf = 0; t0 < hi; t0 += TC, buf ^= 1) {
    if (t0 + TC < hi) ask(t0 + TC);
    const int nt = min(TC, hi - t0);
    for (int tt = 0; tt < nt; ++tt) {
      const float gt = gs[buf][tt], bt = bs[buf][tt], vt = vs[buf][tt * SCAN_COLS + col];
      const float* kt = &ks[buf][tt * KD + part * KQ];
      const float* qt = &qs[buf][tt * KD + part * KQ];
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < KQ; ++i) {
        S[i] *= gt;
        dot += S[i] * kt[i];
      }
      const float u = bt * (vt - part_sum(dot));
      if (local) {
#pragma unroll
        for (int i = 0; i < KQ; ++i) S[i] += kt[i] * u;
        continue;
      }
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < KQ; ++i) {
        S[i] += kt[i] * u;
        o += S[i] * qt[i];
      }
      o = part_sum(o);
      if (active && part == 0) out[((int64_t)(t0 + tt) * heads + h) * vdim + j] = o;
    }
    if (t0 + TC < hi) put(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int row = part * KQ + i;
    if (!active || row >= dim) continue;
    if (local) pc.ab[((piece_no * heads + h) * dim + row) * (int64_t)(vdim + dim) + j] = S[i];
    else if (to_slot) held[(int64_t)row * vdim + j] = S[i];
  }
}

// Between the two passes: a row's pieces in order, S <- A S + B, sixteen columns of S a block (columns never meet).
// A comes through LDS in slabs of 32 columns, S's sixteen columns stay there. sin[p] becomes the state piece p + 1
// starts from.
__global__ void __launch_bounds__(256) delta_pieces_kernel(const float* __restrict__ state,
                                                           const int32_t* __restrict__ slots,
                                                           const int32_t* __restrict__ starts,
                                                           const int32_t* __restrict__ query_start, int heads, int dim,
                                                           int vdim, DeltaPieces pc) {
  constexpr int SLAB = 32, MAXD = 256, PER = MAXD * 16 / 256;
  __shared__ float sc[MAXD * 16];
  __shared__ float as[MAXD][SLAB + 1];
  const int b = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * 16;
  const int pieces = (query_start[b + 1] - query_start[b] + pc.tokens - 1) / pc.tokens;
  const float* held = state + ((int64_t)slots[b] * heads + h) * dim * vdim;
  const bool carried = starts[b] > 0;
  for (int e = threadIdx.x; e < MAXD * 16; e += 256) {      // (rows from dim on stay zero: the slabs reach past dim)
    const int m = e / 16, j = j0 + e % 16;
    sc[e] = carried && m < dim && j < vdim ? held[(int64_t)m * vdim + j] : 0.f;
  }
  for (int e = dim * SLAB + threadIdx.x; e < MAXD * SLAB; e += 256) as[e / SLAB][e % SLAB] = 0.f;   // rows no slab fills
  const int c = threadIdx.x % 16;                            // this thread's column of the sixteen, whatever k
  for (int p = 0; p + 1 < pieces; ++p) {
    const int64_t at = ((int64_t)pc.base[b] + p) * heads + h;
    const float* ab = pc.ab + at * dim * (vdim + dim);
    float* next = pc.sin + at * dim * vdim;
    float acc[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) {                      // element e = threadIdx.x + 256 k: row e / 16, column e % 16
      const int e = threadIdx.x + 256 * k, i = e / 16, j = j0 + e % 16;
      acc[k] = e < dim * 16 && j < vdim ? ab[(int64_t)i * (vdim + dim) + j] : 0.f;
    }
    for (int m0 = 0; m0 < dim; m0 += SLAB) {
      __syncthreads();                                   // the slab before, and S, are settled
      float slab[MAXD * SLAB / 256];                     // all of a thread's loads under way before the first is used
#pragma unroll
      for (int k = 0; k < MAXD * SLAB / 256; ++k) {
        const int e = threadIdx.x + 256 * k, i = e / SLAB, m = e % SLAB;
        slab[k] = e < dim * SLAB && m0 + m < dim ? ab[(int64_t)i * (vdim + dim) + vdim + m0 + m] : 0.f;
      }
#pragma unroll
      for (int k = 0; k < MAXD * SLAB / 256; ++k) {
        const int e = threadIdx.x + 256 * k;
        if (e < dim * SLAB) as[e / SLAB][e % SLAB] = slab[k];
      }
      __syncthreads();
#pragma unroll
      for (int m = 0; m < SLAB; ++m) {                   // (A is zero past dim, and so are S's rows there)
        const float sv = sc[(m0 + m) * 16 + c];
#pragma unroll
        for (int k = 0; k < PER; ++k) acc[k] += as[threadIdx.x / 16 + 16 * k][m] * sv;
      }
    }
    __syncthreads();                                     // every thread has read the old S
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int e = threadIdx.x + 256 * k, i = e / 16, j = j0 + e % 16;
      if (e < dim * 16) {
        sc[e] = acc[k];
        if (j < vdim) next[(int64_t)i * vdim + j] = acc[k];
      }
    }
  }
}

// A long row's tokens in pieces that run side by side (the memory's recurrence is linear in S and its decays do not
// depend on S): every piece but a row's last first runs from S = 0 and leaves what it adds (`sloc`) and the product of
// its decays per key row (`pw`); a small kernel then walks a row's pieces in order, S <- diag(pw) S + sloc, leaving
// each piece's true starting state in place of `sloc`; then every piece runs again from there and writes its outputs.
struct ScanPieces {
  int tokens;                  // tokens a piece (0: rows are not cut)
  int mode;                    // 1: from zero, leave sloc and pw; 2: from the true start, write outputs
  const int32_t* base;         // [rows]: the number of row b's first piece among all pieces of the step
  float* sloc;                 // [pieces, H, D, D]
  float* pw;                   // [pieces, H, D]
};

// Per (row, head): o = (S + diag(u) k v^T)^T r; S <- diag(w) S + k v^T. The same split of S [D, D] over lanes.
template <int KD, typename T>
__global__ void __launch_bounds__(WAVE) memory_scan_kernel(const T* __restrict__ r, const T* __restrict__ k,
                                                           const T* __restrict__ v, const float* __restrict__ w,
                                                           const float* __restrict__ u, float* __restrict__ state,
                                                           float* __restrict__ out, const int32_t* __restrict__ slots,
                                                           const int32_t* __restrict__ starts,
                                                           const int32_t* __restrict__ query_start, int heads, int dim,
                                                           ScanPieces pc) {
  constexpr int KQ = KD / SCAN_PARTS, TC = ScanChunk<KD, 3>::kTokens, N = TC * KD, PER = (N + WAVE - 1) / WAVE;
  constexpr int VPER = (TC * SCAN_COLS + WAVE - 1) / WAVE;
  __shared__ __attribute__((aligned(16))) float rs[2][N], ks[2][N], ws[2][N], us[KD];
  __shared__ float vs[2][TC * SCAN_COLS];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int col_blocks = (dim + SCAN_COLS - 1) / SCAN_COLS;
  const int piece = blockIdx.z / col_blocks, col_block = blockIdx.z % col_blocks;
  const int part = lane % SCAN_PARTS, col = lane / SCAN_PARTS, j = col_block * SCAN_COLS + col;
  const bool active = j < dim;
  int lo = query_start[b], hi = query_start[b + 1];
  bool from_slot = true, to_slot = true;
  int64_t piece_no = 0;
  if (pc.tokens > 0) {                                   // (everything here is the same in all of the block's lanes)
    const int pieces = (hi - lo + pc.tokens - 1) / pc.tokens;
    if (piece >= pieces || (pc.mode == 1 && piece == pieces - 1)) return;
    lo += piece * pc.tokens;
    hi = min(hi, lo + pc.tokens);
    from_slot = piece == 0;
    to_slot = pc.mode == 2 && piece == pieces - 1;
    piece_no = pc.base[b] + piece;
  }
  float* held = state + ((int64_t)slots[b] * heads + h) * dim * dim;
  const bool carried = starts[b] > 0;
  float S[KQ], pw[KQ];
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int row = part * KQ + i;
    const bool in = active && row < dim;
    pw[i] = 1.f;
    if (pc.tokens > 0 && pc.mode == 1) S[i] = 0.f;
    else if (from_slot) S[i] = (carried && in) ? held[(int64_t)row * dim + j] : 0.f;
    else S[i] = in ? pc.sloc[((piece_no - 1) * heads + h) * dim * dim + (int64_t)row * dim + j] : 0.f;
  }
  for (int i = lane; i < KD; i += WAVE) us[i] = i < dim ? u[h * dim + i] : 0.f;
  const int64_t width = (int64_t)heads * dim;
  float nr[PER], nk[PER], nw[PER], nv[VPER];
  auto ask = [&](int t0) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = lane + e * WAVE, tt = idx / KD, i = idx - tt * KD;
      const bool ok = idx < N && t0 + tt < hi && i < dim;
      const int64_t at = (int64_t)(t0 + tt) * width + h * dim + i;
      nr[e] = ok ? Elem<T>::load(r[at]) : 0.f;
      nk[e] = ok ? Elem<T>::load(k[at]) : 0.f;
      nw[e] = ok ? w[at] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < VPER; ++e) {
      const int idx = lane + e * WAVE, tt = idx / SCAN_COLS, jj = col_block * SCAN_COLS + idx % SCAN_COLS;
      const bool ok = idx < TC * SCAN_COLS && t0 + tt < hi && jj < dim;
      nv[e] = ok ? Elem<T>::load(v[(int64_t)(t0 + tt) * width + h * dim + jj]) : 0.f;
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = lane + e * WAVE;
      if (idx < N) { rs[buf][idx] = nr[e]; ks[buf][idx] = nk[e]; ws[buf][idx] = nw[e]; }
    }
#pragma unroll
    for (int e = 0; e < VPER; ++e) {
      const int idx = lane + e * WAVE;
      if (idx < TC * SCAN_COLS) vs[buf][idx] = nv[e];
    }
  };
  if (lo < hi) {
    ask(lo);
    put(0);
  }
  __syncthreads();
  const bool local = pc.tokens > 0 && pc.mode == 1;
  for (int t0 = lo, buf = 0; t0 < hi; t0 += TC, buf ^= 1) {
    if (t0 + TC < hi) ask(t0 + TC);
    const int nt = min(TC, hi - t0);
    for (int tt = 0; tt < nt; ++tt) {
      const float vt = vs[buf][tt * SCAN_COLS + col];
      const float* rt = &rs[buf][tt * KD + part * KQ];
      const float* kt = &ks[buf][tt * KD + part * KQ];
      const float* wt = &ws[buf][tt * KD + part * KQ];
      const float* ut = &us[part * KQ];
      if (local) {                       // what the piece adds to S, and its decays' product; no output yet
#pragma unroll
        for (int i = 0; i < KQ; ++i) {
          S[i] = wt[i] * S[i] + kt[i] * vt;
          pw[i] *= wt[i];
        }
        continue;
      }
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < KQ; ++i) {
        const float kv = kt[i] * vt;
        o += rt[i] * (S[i] + ut[i] * kv);
        S[i] = wt[i] * S[i] + kv;
      }
      o = part_sum(o);
      if (active && part == 0) out[(int64_t)(t0 + tt) * width + h * dim + j] = o;
    }
    if (t0 + TC < hi) put(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int row = part * KQ + i;
    if (!active || row >= dim) continue;
    if (local) {
      pc.sloc[(piece_no * heads + h) * dim * dim + (int64_t)row * dim + j] = S[i];
      if (j == 0) pc.pw[(piece_no * heads + h) * dim + row] = pw[i];
    } else if (to_slot) {
      held[(int64_t)row * dim + j] = S[i];
    }
  }
}

// Between the two passes: a row's pieces in order. sloc[p] becomes the state piece p + 1 starts from.
__global__ void __launch_bounds__(256) memory_pieces_kernel(const float* __restrict__ state,
                                                            const int32_t* __restrict__ slots,
                                                            const int32_t* __restrict__ starts,
                                                            const int32_t* __restrict__ query_start, int heads, int dim,
                                                            ScanPieces pc) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int pieces = (query_start[b + 1] - query_start[b] + pc.tokens - 1) / pc.tokens;
  const float* held = state + ((int64_t)slots[b] * heads + h) * dim * dim;
  const bool carried = starts[b] > 0;
  for (int e = threadIdx.x; e < dim * dim; e += 256) {
    const int row = e / dim;
    float s = carried ? held[e] : 0.f;
    for (int p = 0; p + 1 < pieces; ++p) {
      const int64_t at = (int64_t)pc.base[b] + p;
      float* add = pc.sloc + (at * heads + h) * dim * dim + e;
      s = pc.pw[(at * heads + h) * dim + row] * s + *add;
      *add = s;
    }
  }
}

// One wave per (token, head): o / sqrt(mean(o^2) + eps) * weight * act(gate), act = silu, or the sigmoid alone
// (`plain_sigmoid`). A token's gates are `gate_stride` values apart (columns of a wider projection). With `den`
// (one value a token and head) o is divided by it first.
template <typename T>
__global__ void __launch_bounds__(256) gated_out_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                        const T* __restrict__ weight, T* __restrict__ y, int64_t cells,
                                                        int heads, int vdim, int per_head, float eps,
                                                        int64_t gate_stride, int plain_sigmoid,
                                                        const float* __restrict__ den) {
  const int64_t cell = (int64_t)blockIdx.x * 4 + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (cell >= cells) return;
  const int h = (int)(cell % heads);
  const float* src = o + cell * vdim;
  const float under = den ? den[cell] : 1.f;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += WAVE) {
    const float v = den ? src[d] / under : src[d];
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)vdim + eps);
  for (int d = lane; d < vdim; d += WAVE) {
    const float wv = Elem<T>::load(weight[per_head ? h * vdim + d : d]);
    const float gv = Elem<T>::load(gate[(cell / heads) * gate_stride + (int64_t)h * vdim + d]);
    const float act = plain_sigmoid ? 1.0f / (1.0f + expf(-gv)) : silu<T>(gv);
    y[cell * vdim + d] = Elem<T>::store((den ? src[d] / under : src[d]) * r * wv * act);
  }
}

template <typename T>
__global__ void shift_mix_kernel(const T* __restrict__ x, const T* __restrict__ mu, T* __restrict__ state,
                                 T* __restrict__ y, const int32_t* __restrict__ slots, const int32_t* __restrict__ starts,
                                 const int32_t* __restrict__ query_start, const int32_t* __restrict__ token_row,
                                 int tokens, int width, int mixes, int keep) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int t = blockIdx.y;
  if (c >= width) return;
  const int b = keep ? t : token_row[t];               // keep: every row has one token, token t is row t
  float prev = 0.f;
  if (!keep && t > query_start[b]) prev = Elem<T>::load(x[(int64_t)(t - 1) * width + c]);
  else if (starts[b] > 0) prev = Elem<T>::load(state[(int64_t)slots[b] * width + c]);
  const float cur = Elem<T>::load(x[(int64_t)t * width + c]);
  for (int s = 0; s < mixes; ++s)
    y[((int64_t)s * tokens + t) * width + c] = Elem<T>::store(cur + (prev - cur) * Elem<T>::load(mu[(int64_t)s * width + c]));
  if (keep) state[(int64_t)slots[b] * width + c] = x[(int64_t)t * width + c];
}

template <typename T>
__global__ void shift_keep_kernel(const T* __restrict__ x, T* __restrict__ state, const int32_t* __restrict__ slots,
                                  const int32_t* __restrict__ query_start, int width) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int b = blockIdx.y;
  if (c >= width) return;
  state[(int64_t)slots[b] * width + c] = x[(int64_t)(query_start[b + 1] - 1) * width + c];
}

// exp(-exp(tanh(a) w2^T + w0)): a block takes 8 tokens and 256 channels; the tokens' tanh values are shared through
// LDS, and w2 comes transposed ([rank, channels]) so that a wave's loads are contiguous and serve all 8 tokens.
constexpr int LORA_TOKENS = 8, LORA_MAX_RANK = 1024;
template <typename T>
__global__ void __launch_bounds__(256) decay_lora_kernel(const float* __restrict__ a, const T* __restrict__ w2t,
                                                         const float* __restrict__ w0, float* __restrict__ y, int tokens,
                                                         int channels, int rank) {
  __shared__ float th[LORA_TOKENS][LORA_MAX_RANK];
  const int t0 = blockIdx.x * LORA_TOKENS;
  const int c = blockIdx.y * 256 + threadIdx.x;
  for (int e = threadIdx.x; e < LORA_TOKENS * rank; e += 256) {
    const int tt = e / rank, r = e - tt * rank;
    th[tt][r] = t0 + tt < tokens ? tanhf(a[(int64_t)(t0 + tt) * rank + r]) : 0.f;
  }
  __syncthreads();
  if (c >= channels) return;
  float acc[LORA_TOKENS];
#pragma unroll
  for (int tt = 0; tt < LORA_TOKENS; ++tt) acc[tt] = 0.f;
  for (int r = 0; r < rank; ++r) {
    const float wv = Elem<T>::load(w2t[(int64_t)r * channels + c]);
#pragma unroll
    for (int tt = 0; tt < LORA_TOKENS; ++tt) acc[tt] += th[tt][r] * wv;
  }
  const float off = w0[c];
#pragma unroll
  for (int tt = 0; tt < LORA_TOKENS; ++tt)
    if (t0 + tt < tokens) y[(int64_t)(t0 + tt) * channels + c] = expf(-expf(acc[tt] + off));
}

}  // namespace

#define BY_DTYPE(dtype, CALL)                    \
  do {                                           \
    if ((dtype) == HOLON_F32) { using T = float; CALL; } \
    else { using T = bf16_t; CALL; }             \
  } while (0)

extern "C" int holon_causal_conv(const void* x, const void* w, void* state, void* y, const int32_t* slots,
                                 const int32_t* starts, const int32_t* query_start, const int32_t* token_row,
                                 int tokens, int rows, int channels, int taps, int state_slots, int add_input, int act,
                                 int dtype, int rows_in_order, void* stream) {
  HOLON_CHECK(tokens >= 0 && rows >= 0 && channels > 0 && taps >= 1 && taps <= 16 && state_slots > 0,
              "causal_conv: tokens=%d rows=%d channels=%d taps=%d", tokens, rows, channels, taps);
  HOLON_CHECK(tokens <= 65535 && rows <= 65535, "causal_conv: %d tokens in %d rows exceed one launch", tokens, rows);
  if (tokens == 0 || rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 block(256), grid_t((channels + 255) / 256, tokens), grid_b((channels + 255) / 256, rows);
  HOLON_CHECK(!rows_in_order || tokens == rows, "causal_conv: rows in order means one token a row, got %d in %d", tokens,
              rows);
  const int vec = dtype == HOLON_F32 ? 4 : 8;
  if (!rows_in_order && channels % vec == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0 &&
      (uintptr_t)state % 16 == 0) {
    const dim3 grid_w((channels / vec + 255) / 256, tokens);
    BY_DTYPE(dtype, (causal_conv_wide_kernel<T><<<grid_w, block, 0, s>>>((const T*)x, (const T*)w, (const T*)state, (T*)y,
                                                                         slots, starts, query_start, token_row,
                                                                         channels, taps, add_input, act)));
  } else {
    BY_DTYPE(dtype, (causal_conv_kernel<T><<<grid_t, block, 0, s>>>((const T*)x, (const T*)w, (T*)state, (T*)y, slots,
                                                                    starts, query_start, token_row, channels, taps,
                                                                    add_input, act, rows_in_order)));
  }
  HOLON_LAUNCH_OK();
  if (taps > 1 && !rows_in_order) {
    BY_DTYPE(dtype, (causal_conv_keep_kernel<T><<<grid_b, block, 0, s>>>((const T*)x, (T*)state, slots, starts,
                                                                         query_start, channels, taps)));
    HOLON_LAUNCH_OK();
  }
  return 0;
}

extern "C" int holon_delta_prepare(const void* qkv, const void* ab, const float* a_log, const float* dt_bias, float* qn,
                                   float* kn, float* beta, float* g, int tokens, int heads, int kv_heads, int dim,
                                   int vdim, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0,
              "delta_prepare: %d/%d heads of %d/%d", heads, kv_heads, dim, vdim);
  if (tokens == 0) return 0;
  BY_DTYPE(dtype, (delta_prepare_kernel<T><<<tokens, 256, 0, (hipStream_t)stream>>>(
                      (const T*)qkv, (const T*)ab, a_log, dt_bias, qn, kn, beta, g, heads, kv_heads, dim, vdim)));
  HOLON_LAUNCH_OK();
  return 0;
}

template <typename T, int KD>
static void launch_delta(dim3 grid, hipStream_t s, const float* qn, const float* kn, const void* qkv,
                         int stride, int voff, const float* beta, const float* g, float* state, float* out,
                         const int32_t* slots, const int32_t* starts, const int32_t* qs, int heads, int kv_heads, int dim,
                         int vdim, DeltaPieces pc) {
  delta_scan_kernel<KD, T><<<grid, WAVE, 0, s>>>(qn, kn, (const T*)qkv, stride, voff, beta, g, state, out, slots,
                                                    starts, qs, heads, kv_heads, dim, vdim, pc);
}

#define BY_KEY_SIZE(dim, CALL)                                  \
  do {                                                          \
    if ((dim) <= 16) { constexpr int KD = 16; CALL; }           \
    else if ((dim) <= 32) { constexpr int KD = 32; CALL; }      \
    else if ((dim) <= 48) { constexpr int KD = 48; CALL; }      \
    else if ((dim) <= 64) { constexpr int KD = 64; CALL; }      \
    else if ((dim) <= 96) { constexpr int KD = 96; CALL; }      \
    else if ((dim) <= 128) { constexpr int KD = 128; CALL; }    \
    else if ((dim) <= 192) { constexpr int KD = 192; CALL; }    \
    else { constexpr int KD = 256; CALL; }                      \
  } while (0)

extern "C" int holon_delta_scan(const float* qn, const float* kn, const void* qkv, int qkv_stride, int v_offset,
                                const float* beta, const float* g, float* state, float* out, const int32_t* slots,
                                const int32_t* starts, const int32_t* query_start, int rows, int heads, int kv_heads,
                                int dim, int vdim, int state_slots, int dtype, int piece_tokens, int max_pieces,
                                const int32_t* piece_base, float* ab, float* sin, void* stream) {
  HOLON_CHECK(rows >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "delta_scan: %d/%d heads", heads, kv_heads);
  HOLON_CHECK(dim > 0 && dim <= 256 && vdim > 0 && vdim <= 1024, "delta_scan: key size %d (at most 256), value size %d "
              "(at most 1024)", dim, vdim);
  HOLON_CHECK(rows <= 0x7fffffff / 2 && heads <= 65535 && state_slots > 0 && v_offset >= 0 &&
              v_offset + heads * vdim <= qkv_stride, "delta_scan: launch or row layout out of range");
  HOLON_CHECK(piece_tokens == 0 || (piece_tokens > 0 && max_pieces > 0 && piece_base && ab && sin),
              "delta_scan: rows in pieces of %d tokens need the pieces' table and workspace", piece_tokens);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  DeltaPieces pc{piece_tokens, 0, piece_base, ab, sin};
  const int col_blocks = (vdim + SCAN_COLS - 1) / SCAN_COLS;     // a wave for every 8 value columns
  if (piece_tokens == 0) {
    const dim3 grid(rows, heads, col_blocks);
    BY_DTYPE(dtype, BY_KEY_SIZE(dim, (launch_delta<T, KD>(grid, s, qn, kn, qkv, qkv_stride, v_offset, beta, g, state,
                                                           out, slots, starts, query_start, heads, kv_heads, dim, vdim,
                                                           pc))));
    HOLON_LAUNCH_OK();
    return 0;
  }
  const int col_blocks_first = (vdim + dim + SCAN_COLS - 1) / SCAN_COLS;
  HOLON_CHECK((int64_t)col_blocks_first * max_pieces <= 65535, "delta_scan: %d pieces a row exceed one launch", max_pieces);
  pc.mode = 1;
  BY_DTYPE(dtype, BY_KEY_SIZE(dim, (launch_delta<T, KD>(dim3(rows, heads, col_blocks_first * max_pieces), s, qn, kn, qkv,
                                                         qkv_stride, v_offset, beta, g, state, out, slots, starts,
                                                         query_start, heads, kv_heads, dim, vdim, pc))));
  HOLON_LAUNCH_OK();
  delta_pieces_kernel<<<dim3(rows, heads, (vdim + 15) / 16), 256, 0, s>>>(state, slots, starts, query_start, heads, dim,
                                                                          vdim, pc);
  HOLON_LAUNCH_OK();
  pc.mode = 2;
  BY_DTYPE(dtype, BY_KEY_SIZE(dim, (launch_delta<T, KD>(dim3(rows, heads, col_blocks * max_pieces), s, qn, kn, qkv,
                                                         qkv_stride, v_offset, beta, g, state, out, slots, starts,
                                                         query_start, heads, kv_heads, dim, vdim, pc))));
  HOLON_LAUNCH_OK();
  return 0;
}

template <typename T, int KD>
static void launch_memory(dim3 grid, hipStream_t s, const void* r, const void* k, const void* v,
                          const float* w, const float* u, float* state, float* out, const int32_t* slots,
                          const int32_t* starts, const int32_t* qs, int heads, int dim, ScanPieces pc) {
  memory_scan_kernel<KD, T><<<grid, WAVE, 0, s>>>((const T*)r, (const T*)k, (const T*)v, w, u, state, out, slots,
                                                     starts, qs, heads, dim, pc);
}

extern "C" int holon_memory_scan(const void* r, const void* k, const void* v, const float* w, const float* u,
                                 float* state, float* out, const int32_t* slots, const int32_t* starts,
                                 const int32_t* query_start, int rows, int heads, int dim, int state_slots, int dtype,
                                 int piece_tokens, int max_pieces, const int32_t* piece_base, float* sloc, float* pw,
                                 void* stream) {
  HOLON_CHECK(rows >= 0 && heads > 0 && heads <= 65535 && dim > 0 && dim <= 256 && state_slots > 0,
              "memory_scan: %d heads of %d (at most 256)", heads, dim);
  HOLON_CHECK(piece_tokens == 0 || (piece_tokens > 0 && max_pieces > 0 && piece_base && sloc && pw),
              "memory_scan: rows in pieces of %d tokens need the pieces' table and workspace", piece_tokens);
  if (rows == 0) return 0;
  const int col_blocks = (dim + SCAN_COLS - 1) / SCAN_COLS;
  hipStream_t s = (hipStream_t)stream;
  ScanPieces pc{piece_tokens, 0, piece_base, sloc, pw};
  if (piece_tokens == 0) {
    const dim3 grid(rows, heads, col_blocks);
    BY_DTYPE(dtype, BY_KEY_SIZE(dim, (launch_memory<T, KD>(grid, s, r, k, v, w, u, state, out, slots, starts,
                                                            query_start, heads, dim, pc))));
    HOLON_LAUNCH_OK();
    return 0;
  }
  HOLON_CHECK((int64_t)col_blocks * max_pieces <= 65535, "memory_scan: %d pieces a row exceed one launch", max_pieces);
  const dim3 grid(rows, heads, col_blocks * max_pieces);
  pc.mode = 1;
  BY_DTYPE(dtype, BY_KEY_SIZE(dim, (launch_memory<T, KD>(grid, s, r, k, v, w, u, state, out, slots, starts,
                                                          query_start, heads, dim, pc))));
  HOLON_LAUNCH_OK();
  memory_pieces_kernel<<<dim3(rows, heads), 256, 0, s>>>(state, slots, starts, query_start, heads, dim, pc);
  HOLON_LAUNCH_OK();
  pc.mode = 2;
  BY_DTYPE(dtype, BY_KEY_SIZE(dim, (launch_memory<T, KD>(grid, s, r, k, v, w, u, state, out, slots, starts,
                                                          query_start, heads, dim, pc))));
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_gated_out(const float* o, const void* gate, const void* weight, void* y, int tokens, int heads,
                               int vdim, int per_head, float eps, int dtype, int64_t gate_stride, int plain_sigmoid,
                               const float* den, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && vdim > 0 && gate_stride >= (int64_t)heads * vdim,
              "gated_out: %d heads of %d, gates %lld apart", heads, vdim, (long long)gate_stride);
  const int64_t cells = (int64_t)tokens * heads;
  if (cells == 0) return 0;
  HOLON_CHECK((cells + 3) / 4 <= 0x7fffffff, "gated_out: %lld cells exceed one launch", (long long)cells);
  BY_DTYPE(dtype, (gated_out_kernel<T><<<(unsigned)((cells + 3) / 4), 256, 0, (hipStream_t)stream>>>(
                      o, (const T*)gate, (const T*)weight, (T*)y, cells, heads, vdim, per_head, eps, gate_stride,
                      plain_sigmoid, den)));
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_shift_mix(const void* x, const void* mu, void* state, void* y, const int32_t* slots,
                               const int32_t* starts, const int32_t* query_start, const int32_t* token_row, int tokens,
                               int rows, int width, int mixes, int state_slots, int dtype, int rows_in_order,
                               void* stream) {
  HOLON_CHECK(tokens >= 0 && rows >= 0 && width > 0 && mixes > 0 && state_slots > 0, "shift_mix: tokens=%d width=%d",
              tokens, width);
  HOLON_CHECK(tokens <= 65535 && rows <= 65535, "shift_mix: %d tokens in %d rows exceed one launch", tokens, rows);
  if (tokens == 0 || rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 block(256), grid_t((width + 255) / 256, tokens), grid_b((width + 255) / 256, rows);
  HOLON_CHECK(!rows_in_order || tokens == rows, "shift_mix: rows in order means one token a row, got %d in %d", tokens,
              rows);
  BY_DTYPE(dtype, (shift_mix_kernel<T><<<grid_t, block, 0, s>>>((const T*)x, (const T*)mu, (T*)state, (T*)y, slots, starts,
                                                                query_start, token_row, tokens, width, mixes,
                                                                rows_in_order)));
  HOLON_LAUNCH_OK();
  if (rows_in_order) return 0;                           // the one kernel has kept each row's token
  BY_DTYPE(dtype, (shift_keep_kernel<T><<<grid_b, block, 0, s>>>((const T*)x, (T*)state, slots, query_start, width)));
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_decay_lora(const float* a, const void* w2t, const float* w0, float* y, int tokens, int channels,
                                int rank, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && channels > 0 && rank > 0 && rank <= LORA_MAX_RANK,
              "decay_lora: %d channels, rank %d (at most %d)", channels, rank, LORA_MAX_RANK);
  if (tokens == 0) return 0;
  const dim3 grid((tokens + LORA_TOKENS - 1) / LORA_TOKENS, (channels + 255) / 256);
  HOLON_CHECK(grid.y <= 65535, "decay_lora: %d channels exceed one launch", channels);
  BY_DTYPE(dtype, (decay_lora_kernel<T><<<grid, 256, 0, (hipStream_t)stream>>>(a, (const T*)w2t, w0, y, tokens, channels,
                                                                               rank)));
  HOLON_LAUNCH_OK();
  return 0;
}
