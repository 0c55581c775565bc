// Kernels around mixers that convolve their projections over a few tokens, gate their outputs, or carry a
// gated linear recurrence per channel; and the small row operations of a layer whose norm sits behind the sublayer.
//
//   causal_conv:   y_t[c] = sum_j w[c][j] * u_(t - taps + 1 + j)[c] (+ bias[c]); the last taps-1 inputs of every request
//                  live in its state slot, so a portion of any length continues where the last one stopped
//   pair_rope_unit: rotation of neighbouring pairs (2i, 2i+1) of the first rot elements of each head at the row's
//                  position, optional division by the head's root mean square, the cache write (keys and values padded
//                  with zeros to the cache's head size) and the queries' copy
//   gate_mul:      out = a * sigmoid(g), heads compacted from the attention's head size to the value size
//   rglru_scan:    S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with a_t = exp(c r_t), r and i sigmoids of block-diagonal
//                  projections of u; out = S_t * gelu_tanh(y_t)
//   norm_add:      x += y / sqrt(mean(y^2) + eps) * w (and, if asked, the new x once more rounded to bfloat16)
//   softcap:       x = cap * tanh(x / cap)
//
// All arithmetic is 32-bit; only stores into a bfloat16 buffer round.  A request without rows, with a negative slot or
// a negative first position is padding and leaves its state alone.
#include <math.h>

#include "common.h"
#include "api.h"

template <typename T> __device__ __forceinline__ float gm_load(const T* p);
template <> __device__ __forceinline__ float gm_load<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float gm_load<bf16_t>(const bf16_t* p) { return bf16_to_f32(*p); }
__device__ __forceinline__ void gm_store(float* p, float v) { *p = v; }
__device__ __forceinline__ void gm_store(bf16_t* p, float v) { *p = f32_to_bf16(v); }

__device__ __forceinline__ float gm_sigmoid(float x) { return 1.0f / (1.0f + bw_expf(-x)); }

// ------------------------------------------------------------------------------ short causal convolution

#define CONV_CHUNK 32
#define CONV_MAX_TAPS 8

struct ConvArgs {
  const float* x;        // [rows, ldx]: channel c at column c
  const void* w;         // [channels, taps]
  const void* bias;      // [channels] or null: added to every output
  const float* in_bias;  // [channels] or null: added to every input on its way in (the state keeps inputs with it)
  float* state;          // [slots, state_ld]: [taps - 1][channels] at the pointer, oldest first
  float* out;            // [rows, ldo]
  const int32_t* seq_rows;
  const int32_t* slots;
  const int32_t* positions;
  long long state_ld;
  int ldx, ldo, channels;
};

template <int TAPS, typename WT>
__global__ __launch_bounds__(256) void causal_conv_kernel(ConvArgs a) {
  constexpr int P = TAPS > 1 ? TAPS - 1 : 1;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int seq = blockIdx.y, t0 = blockIdx.z * CONV_CHUNK;
  const int first = a.seq_rows[2 * seq], n = a.seq_rows[2 * seq + 1], slot = a.slots[seq];
  if (c >= a.channels || n <= 0 || slot < 0 || t0 >= n || a.positions[first] < 0) return;
  const int t1 = min(n, t0 + CONV_CHUNK);
  float w[TAPS];
#pragma unroll
  for (int j = 0; j < TAPS; ++j) w[j] = gm_load(reinterpret_cast<const WT*>(a.w) + (size_t)c * TAPS + j);
  const float bias = a.bias != nullptr ? gm_load(reinterpret_cast<const WT*>(a.bias) + c) : 0.0f;
  float* st = a.state + (size_t)slot * a.state_ld + c;
  const float* x = a.x + (size_t)first * a.ldx + c;
  const float ib = a.in_bias != nullptr ? a.in_bias[c] : 0.0f;
  // only the request's first chunk reaches back before the portion, and only its threads touch the slot
  float old[P];
#pragma unroll
  for (int j = 0; j < P; ++j) old[j] = (TAPS > 1 && t0 == 0) ? st[(size_t)j * a.channels] : 0.0f;
  float win[P];
#pragma unroll
  for (int j = 0; j < P; ++j) {
    const int idx = t0 - (TAPS - 1) + j;
    win[j] = idx >= 0 ? x[(size_t)idx * a.ldx] + ib : old[(TAPS - 1 + idx) < 0 ? 0 : (TAPS - 1 + idx)];
  }
  float* o = a.out + (size_t)first * a.ldo + c;
  for (int t = t0; t < t1; ++t) {
    const float cur = x[(size_t)t * a.ldx] + ib;
    float acc = 0.0f;
    if constexpr (TAPS > 1) {
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j) acc = fmaf(w[j], win[j], acc);
    }
    acc = fmaf(w[TAPS - 1], cur, acc);
    if (a.bias != nullptr) acc += bias;
    o[(size_t)t * a.ldo] = acc;
    if constexpr (TAPS > 1) {
#pragma unroll
      for (int j = 0; j + 1 < TAPS - 1; ++j) win[j] = win[j + 1];
      win[TAPS - 2] = cur;
    }
  }
  if (TAPS > 1 && t0 == 0) {
#pragma unroll
    for (int j = 0; j < TAPS - 1; ++j) {
      const int idx = n - (TAPS - 1) + j;
      float v = 0.0f;
      if (idx >= 0) v = x[(size_t)idx * a.ldx] + ib;
      else {
#pragma unroll
        for (int q = 0; q < P; ++q) v = (q == TAPS - 1 + idx) ? old[q] : v;
      }
      st[(size_t)j * a.channels] = v;
    }
  }
}

template <typename WT>
static int conv_launch(const ConvArgs& a, int taps, dim3 grid, hipStream_t s) {
  switch (taps) {
#define CONV_CASE(T) case T: hipLaunchKernelGGL((causal_conv_kernel<T, WT>), grid, dim3(256), 0, s, a); break;
    CONV_CASE(1) CONV_CASE(2) CONV_CASE(3) CONV_CASE(4) CONV_CASE(5) CONV_CASE(6) CONV_CASE(7) CONV_CASE(8)
#undef CONV_CASE
    default: return -2;
  }
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_causal_conv(const float* x, int ldx, const float* in_bias, const void* w, const void* bias, int w_is_bf16, int taps, int channels,
                              float* state, long long state_ld, const int32_t* seq_rows, const int32_t* slots,
                              const int32_t* positions, int nseq, int max_seq_rows, float* out, int ldo, void* stream) {
  if (nseq <= 0 || channels <= 0 || max_seq_rows <= 0) return 0;
  if (taps < 1 || taps > CONV_MAX_TAPS || (taps > 1 && state == nullptr)) return -2;
  ConvArgs a{x, w, bias, in_bias, state, out, seq_rows, slots, positions, state_ld, ldx, ldo, channels};
  const dim3 grid((channels + 255) / 256, nseq, (max_seq_rows + CONV_CHUNK - 1) / CONV_CHUNK);
  if (grid.y > 65535 || grid.z > 65535) return -2;
  return w_is_bf16 ? conv_launch<bf16_t>(a, taps, grid, (hipStream_t)stream) : conv_launch<float>(a, taps, grid, (hipStream_t)stream);
}

// ------------------------------------------------------------------------------ pair rotation, unit norm, cache write

struct PairRopeArgs {
  const float* src;            // [rows, lds]: q heads (dim each), then k heads (dim each), then v heads (vdim each)
  const int32_t* positions;
  const int32_t* row_seq;
  const int32_t* block_table;
  const float* cos_table;      // [positions, rot / 2]
  const float* sin_table;
  void* q_out;                 // [rows, heads * hd]
  void* k_cache;
  void* v_cache;
  int lds, rows, heads, kv_heads, dim, vdim, hd, rot, page_size, table_stride, unit_norm, has_kv, write_cache;
  float eps;
  int halves;                  // 0: pair i of the rotation is elements (2i, 2i+1); 1: elements (i, i + rot/2)
  int v_from_k;                // 1: src holds no values; a value head is the key head as projected (vdim == dim)
};

// A wave a (row, head): q heads, then k heads, then v heads.  Lane l owns the pairs l, l + 64, ...
template <typename T>
__global__ __launch_bounds__(256) void pair_rope_unit_kernel(PairRopeArgs a) {
  const int per_row = a.heads + (a.has_kv ? 2 * a.kv_heads : 0);
  const int item = blockIdx.x * 4 + wave_index();
  if (item >= a.rows * per_row) return;
  const int row = item / per_row, hh = item % per_row, lane = threadIdx.x & 63;
  const int pos = a.positions[row];
  if (pos < 0) return;
  const bool is_q = hh < a.heads, is_k = !is_q && hh < a.heads + a.kv_heads;
  if (!is_q && !a.write_cache) return;
  const int page = a.block_table[(size_t)a.row_seq[row] * a.table_stride + pos / a.page_size];
  const int slot = pos % a.page_size;
  if (!is_q && !is_k) {
    // values: as they are, padded with zeros to the cache's head size
    const int h = hh - a.heads - a.kv_heads;
    const float* v = a.v_from_k ? a.src + (size_t)row * a.lds + (size_t)(a.heads + h) * a.dim
                                : a.src + (size_t)row * a.lds + (size_t)(a.heads + a.kv_heads) * a.dim + (size_t)h * a.vdim;
    T* vc = reinterpret_cast<T*>(a.v_cache);
    for (int d = lane; d < a.hd; d += 64) {
      const float val = d < a.vdim ? v[d] : 0.0f;
      if constexpr (sizeof(T) == 2) gm_store(vc + (((size_t)page * a.kv_heads + h) * a.hd + d) * a.page_size + slot, val);   // [kv head][element][slot]
      else gm_store(vc + (((size_t)page * a.kv_heads + h) * a.page_size + slot) * a.hd + d, val);
    }
    return;
  }
  const float* v = a.src + (size_t)row * a.lds + (size_t)hh * a.dim;
  const int half = a.rot / 2, pairs = (a.dim + 1) / 2;
  const float* ct = a.cos_table + (size_t)pos * half;
  const float* st = a.sin_table + (size_t)pos * half;
  // up to 256 elements a head: two pairs a lane
  float e0[2], e1[2];
  float acc = 0.0f;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int p = lane + 64 * j;
    e0[j] = e1[j] = 0.0f;
    if (p < pairs) {
      // (pairs behind the rotated ones are neighbours in either layout)
      const int i1 = a.halves && p < half ? p : 2 * p, i2 = a.halves && p < half ? p + half : 2 * p + 1;
      const float x1 = v[i1], x2 = i2 < a.dim ? v[i2] : 0.0f;
      if (p < half) {
        const float c = ct[p], s = st[p];
        e0[j] = x1 * c - x2 * s;
        e1[j] = x2 * c + x1 * s;
      } else {
        e0[j] = x1;
        e1[j] = x2;
      }
      acc = fmaf(e0[j], e0[j], acc);
      acc = fmaf(e1[j], e1[j], acc);
    }
  }
  float inv = 1.0f;
  if (a.unit_norm) {
    acc = wave_sum(acc);
    inv = 1.0f / sqrtf(acc / (float)a.dim + a.eps);
  }
  T* dst;
  if (is_q) dst = reinterpret_cast<T*>(a.q_out) + (size_t)row * a.heads * a.hd + (size_t)hh * a.hd;
  else dst = reinterpret_cast<T*>(a.k_cache) + (((size_t)page * a.kv_heads + (hh - a.heads)) * a.page_size + slot) * a.hd;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int p = lane + 64 * j;
    const int i1 = a.halves && p < half ? p : 2 * p, i2 = a.halves && p < half ? p + half : 2 * p + 1;
    if (i1 < a.hd) gm_store(dst + i1, i1 < a.dim ? e0[j] * inv : 0.0f);
    if (i2 < a.hd) gm_store(dst + i2, i2 < a.dim ? e1[j] * inv : 0.0f);
  }
}

extern "C" int bw_pair_rope_unit(const float* src, int lds, const int32_t* positions, const int32_t* row_seq,
                                 const int32_t* block_table, int table_stride, const float* cos_table, const float* sin_table,
                                 void* q_out, void* k_cache, void* v_cache, int is_bf16, int rows, int heads, int kv_heads,
                                 int dim, int vdim, int hd, int rot, int page_size, int unit_norm, float eps, int has_kv,
                                 int write_cache, int halves, int v_from_k, void* stream) {
  if (rows <= 0) return 0;
  if (dim > 256 || hd > 256 || dim > hd || vdim > hd || rot % 2 || rot > dim || page_size <= 0) return -2;
  if (v_from_k && vdim != dim) return -2;
  PairRopeArgs a{src, positions, row_seq, block_table, cos_table, sin_table, q_out, k_cache, v_cache, lds, rows, heads, kv_heads,
                 dim, vdim, hd, rot, page_size, table_stride, unit_norm, has_kv, write_cache, eps, halves, v_from_k};
  const long long items = (long long)rows * (heads + (has_kv ? 2 * kv_heads : 0));
  const dim3 grid((unsigned)((items + 3) / 4));
  if (is_bf16) hipLaunchKernelGGL(pair_rope_unit_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, a);
  else hipLaunchKernelGGL(pair_rope_unit_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, a);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ norm over whole projections, value mixing

struct WholeNormArgs {
  const float* src;
  const int32_t* positions;
  const int32_t* row_seq;
  const int32_t* block_table;
  const float* q_w;
  const float* k_w;
  const float* v_first;
  const float* lambda;
  float* v_keep;
  void* q_out;
  void* k_cache;
  void* v_cache;
  int lds, ldf, ldk, heads, kv_heads, dim, vdim, hd, page_size, table_stride, write_cache;
  float eps;
};

// The workgroup's sum of one number a thread: the waves' sums (xor butterflies) added in wave order.
__device__ __forceinline__ float workgroup_sum_256(float v, float* lds4) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
  __syncthreads();
  const float t = ((lds4[0] + lds4[1]) + lds4[2]) + lds4[3];
  __syncthreads();
  return t;
}

// A workgroup for each of a row's three parts (queries, keys, values): each is one chain of loads, a sum and stores.
template <typename T>
__global__ __launch_bounds__(256) void whole_norm_kv_kernel(WholeNormArgs a) {
  __shared__ float red[4];
  const int row = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
  const int pos = a.positions[row];
  if (pos < 0) return;
  const int qn = a.heads * a.dim, kn = a.kv_heads * a.dim;
  const float* q = a.src + (size_t)row * a.lds;
  if (part == 0) {
    float acc = 0.0f;
    for (int i = tid; i < qn; i += 256) acc = fmaf(q[i], q[i], acc);
    const float inv_q = 1.0f / sqrtf(workgroup_sum_256(acc, red) / (float)qn + a.eps);
    T* qo = reinterpret_cast<T*>(a.q_out) + (size_t)row * a.heads * a.hd;
    for (int i = tid; i < a.heads * a.hd; i += 256) {
      const int h = i / a.hd, d = i % a.hd;
      gm_store(qo + i, d < a.dim ? (q[h * a.dim + d] * inv_q) * a.q_w[h * a.dim + d] : 0.0f);
    }
    return;
  }
  if (!a.write_cache) return;
  const int page = a.block_table[(size_t)a.row_seq[row] * a.table_stride + pos / a.page_size];
  const int slot = pos % a.page_size;
  if (part == 1) {
    const float* k = q + qn;
    float acc = 0.0f;
    for (int i = tid; i < kn; i += 256) acc = fmaf(k[i], k[i], acc);
    const float inv_k = 1.0f / sqrtf(workgroup_sum_256(acc, red) / (float)kn + a.eps);
    T* kc = reinterpret_cast<T*>(a.k_cache);
    for (int i = tid; i < a.kv_heads * a.hd; i += 256) {
      const int h = i / a.hd, d = i % a.hd;
      gm_store(kc + (((size_t)page * a.kv_heads + h) * a.page_size + slot) * a.hd + d,
               d < a.dim ? (k[h * a.dim + d] * inv_k) * a.k_w[h * a.dim + d] : 0.0f);
    }
    return;
  }
  const float* v = q + qn + kn;
  T* vc = reinterpret_cast<T*>(a.v_cache);
  const float lam = a.v_first != nullptr ? a.lambda[0] : 0.0f;
  for (int i = tid; i < a.kv_heads * a.hd; i += 256) {
    const int h = i / a.hd, d = i % a.hd;
    float val = 0.0f;
    if (d < a.vdim) {
      val = v[h * a.vdim + d];
      if (a.v_keep != nullptr) a.v_keep[(size_t)row * a.ldk + h * a.vdim + d] = val;
      if (a.v_first != nullptr) val = (1.0f - lam) * val + lam * a.v_first[(size_t)row * a.ldf + h * a.vdim + d];
    }
    if constexpr (sizeof(T) == 2) gm_store(vc + (((size_t)page * a.kv_heads + h) * a.hd + d) * a.page_size + slot, val);   // [kv head][element][slot]
    else gm_store(vc + (((size_t)page * a.kv_heads + h) * a.page_size + slot) * a.hd + d, val);
  }
}

extern "C" int bw_whole_norm_kv(const float* src, int lds, const int32_t* positions, const int32_t* row_seq,
                                const int32_t* block_table, int table_stride, const float* q_w, const float* k_w, float eps,
                                const float* v_first, int ldf, const float* lambda, float* v_keep, int ldk, void* q_out,
                                void* k_cache, void* v_cache, int is_bf16, int rows, int heads, int kv_heads, int dim, int vdim,
                                int hd, int page_size, int write_cache, void* stream) {
  if (rows <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || dim <= 0 || vdim <= 0 || dim > hd || vdim > hd || page_size <= 0) return -2;
  if (lds < heads * dim + (write_cache ? kv_heads * (dim + vdim) : 0)) return -2;
  if (v_first != nullptr && (lambda == nullptr || ldf < kv_heads * vdim)) return -2;
  if (v_keep != nullptr && ldk < kv_heads * vdim) return -2;
  if (v_keep != nullptr && v_keep == v_first) return -2;
  WholeNormArgs a{src, positions, row_seq, block_table, q_w, k_w, v_first, lambda, v_keep, q_out, k_cache, v_cache, lds, ldf, ldk,
                  heads, kv_heads, dim, vdim, hd, page_size, table_stride, write_cache, eps};
  if (is_bf16) hipLaunchKernelGGL(whole_norm_kv_kernel<bf16_t>, dim3(rows, 3), dim3(256), 0, (hipStream_t)stream, a);
  else hipLaunchKernelGGL(whole_norm_kv_kernel<float>, dim3(rows, 3), dim3(256), 0, (hipStream_t)stream, a);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ output gate

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gate_mul_kernel(const TI* __restrict__ av, int lda, int hd, const float* __restrict__ g, int ldg,
                                                       TO* __restrict__ out, int ldo, int rows, int heads, int vdim, int per_head) {
  const int row = blockIdx.y;
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= heads * vdim) return;
  const int h = e / vdim, d = e % vdim;
  const float x = gm_load(av + (size_t)row * lda + (size_t)h * hd + d);
  gm_store(out + (size_t)row * ldo + e, x * gm_sigmoid(g[(size_t)row * ldg + (per_head ? h : e)]));
}

extern "C" int bw_gate_mul(const void* av, int a_is_bf16, int lda, int hd, const float* g, int ldg, void* out, int out_is_bf16,
                           int ldo, int rows, int heads, int vdim, int per_head, void* stream) {
  if (rows <= 0) return 0;
  if (rows > 65535 * 16) return -2;
  const dim3 grid((heads * vdim + 255) / 256, rows);
  hipStream_t s = (hipStream_t)stream;
  if (a_is_bf16 && out_is_bf16)
    hipLaunchKernelGGL((gate_mul_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, s, (const bf16_t*)av, lda, hd, g, ldg, (bf16_t*)out, ldo, rows, heads, vdim, per_head);
  else if (a_is_bf16)
    hipLaunchKernelGGL((gate_mul_kernel<bf16_t, float>), grid, dim3(256), 0, s, (const bf16_t*)av, lda, hd, g, ldg, (float*)out, ldo, rows, heads, vdim, per_head);
  else if (out_is_bf16)
    hipLaunchKernelGGL((gate_mul_kernel<float, bf16_t>), grid, dim3(256), 0, s, (const float*)av, lda, hd, g, ldg, (bf16_t*)out, ldo, rows, heads, vdim, per_head);
  else
    hipLaunchKernelGGL((gate_mul_kernel<float, float>), grid, dim3(256), 0, s, (const float*)av, lda, hd, g, ldg, (float*)out, ldo, rows, heads, vdim, per_head);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ gated linear recurrence per channel

struct RglruArgs {
  const float* y;         // [rows, ldy]: the gate branch before its activation
  const float* u;         // [rows, ldu]: the convolved recurrent branch
  const float* gates;     // [rows, ldg]: per block of bs channels, bs recurrence-gate logits then bs input-gate logits
  const float* ra_bias;   // [channels]
  const float* ri_bias;
  const float* decay;     // [channels]: c = -scale * softplus(lambda), so that log a = c * r
  const float* y_bias;    // [channels] or null: added to the gate branch before its activation
  float* state;           // [slots, state_ld]: S [channels] at the pointer
  void* out;              // [rows, ldo]
  const int32_t* seq_rows;
  const int32_t* slots;
  const int32_t* positions;
  long long state_ld;
  int ldy, ldu, ldg, ldo, channels, bs;
};

__device__ __forceinline__ float gm_gelu_tanh(float z) {
  const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.0f + tanhf(inner));
}

// What a token adds to its channel's state and the factor the state keeps: independent of the state itself.
__device__ __forceinline__ void rglru_terms(float zr, float zi, float u, float br, float bi, float c, float& a, float& b) {
  const float r = gm_sigmoid(zr + br), i = gm_sigmoid(zi + bi);
  const float log_a = c * r;
  a = bw_expf(log_a);
  b = sqrtf(-expm1f(2.0f * log_a)) * (i * u);      // sqrt(1 - a^2) without the cancellation near a = 1
}

// Pass 1, a thread an element (row, channel): the factor a, the addend b and the gate branch's activation, each a
// function of the row alone, over the gates' logits, u and y in place (gates[.., r logits] <- a, gates[.., i logits] <- b,
// y <- gelu_tanh(y)).  Pass 2, a thread a channel of a request: S <- a S + b along the rows in order, out = S * y.
__global__ __launch_bounds__(256) void rglru_terms_kernel(RglruArgs p, int rows) {
  const int c = blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
  if (c >= p.channels || p.positions[row] < 0) return;
  const int blk = c / p.bs, o = c % p.bs;
  float* zr = const_cast<float*>(p.gates) + (size_t)row * p.ldg + (size_t)blk * 2 * p.bs + o;
  float* yy = const_cast<float*>(p.y) + (size_t)row * p.ldy + c;
  float a, b;
  rglru_terms(zr[0], zr[p.bs], p.u[(size_t)row * p.ldu + c], p.ra_bias[c], p.ri_bias[c], p.decay[c], a, b);
  zr[0] = a;
  zr[p.bs] = b;
  *yy = gm_gelu_tanh(p.y_bias != nullptr ? *yy + p.y_bias[c] : *yy);
}

template <typename TO>
__global__ __launch_bounds__(64) void rglru_scan_kernel(RglruArgs p) {
  const int c = blockIdx.x * 64 + threadIdx.x, seq = blockIdx.y;
  const int first = p.seq_rows[2 * seq], n = p.seq_rows[2 * seq + 1], slot = p.slots[seq];
  if (c >= p.channels || n <= 0 || slot < 0 || p.positions[first] < 0) return;
  const int blk = c / p.bs, o = c % p.bs;
  const float* za = p.gates + (size_t)first * p.ldg + (size_t)blk * 2 * p.bs + o;
  const float* zb = za + p.bs;
  const float* y = p.y + (size_t)first * p.ldy + c;
  TO* out = reinterpret_cast<TO*>(p.out) + (size_t)first * p.ldo + c;
  float* st = p.state + (size_t)slot * p.state_ld + c;
  float S = *st;
  constexpr int UN = 16;
  int t = 0;
  for (; t + UN <= n; t += UN) {
    float va[UN], vb[UN], vy[UN];
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      va[j] = za[(size_t)(t + j) * p.ldg];
      vb[j] = zb[(size_t)(t + j) * p.ldg];
      vy[j] = y[(size_t)(t + j) * p.ldy];
    }
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      S = fmaf(va[j], S, vb[j]);
      gm_store(out + (size_t)(t + j) * p.ldo, S * vy[j]);
    }
  }
  for (; t < n; ++t) {
    S = fmaf(za[(size_t)t * p.ldg], S, zb[(size_t)t * p.ldg]);
    gm_store(out + (size_t)t * p.ldo, S * y[(size_t)t * p.ldy]);
  }
  *st = S;
}

extern "C" int bw_rglru_scan(float* y, int ldy, const float* y_bias, const float* u, int ldu, float* gates, int ldg, const float* ra_bias,
                             const float* ri_bias, const float* decay, float* state, long long state_ld, void* out,
                             int out_is_bf16, int ldo, const int32_t* seq_rows, const int32_t* slots, const int32_t* positions,
                             int nseq, int rows, int channels, int bs, void* stream) {
  if (nseq <= 0 || channels <= 0 || rows <= 0) return 0;
  if (bs <= 0 || channels % bs || nseq > 65535 || rows > 65535) return -2;
  RglruArgs p{y, u, gates, ra_bias, ri_bias, decay, y_bias, state, out, seq_rows, slots, positions, state_ld, ldy, ldu, ldg, ldo, channels, bs};
  hipLaunchKernelGGL(rglru_terms_kernel, dim3((channels + 255) / 256, rows), dim3(256), 0, (hipStream_t)stream, p, rows);
  const dim3 grid((channels + 63) / 64, nseq);
  if (out_is_bf16) hipLaunchKernelGGL(rglru_scan_kernel<bf16_t>, grid, dim3(64), 0, (hipStream_t)stream, p);
  else hipLaunchKernelGGL(rglru_scan_kernel<float>, grid, dim3(64), 0, (hipStream_t)stream, p);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ x += rmsnorm(y) * w

// A workgroup a row.  Thread t owns elements t, t + 256, ...; its sum of squares is one chain over them, the waves'
// sums are joined by the butterflies of wave_sum and the four of them added in wave order: the same order for every
// row of every launch.  rounded (optional): the new row once more, rounded to bfloat16, for the next sublayer's products.
// place, wts (optional): y is then not the row itself but a table of rows of which this row is a weighted sum,
// y_row[e] = sum_j wts[row][j] * y[place[row][j]][e], j ascending, one chain an element (what a feed-forward of routed
// experts leaves: its choices' outputs by sorted place); the sum is formed here instead of by a launch of its own.
template <typename WT>
__global__ __launch_bounds__(256) void norm_add_kernel(const float* __restrict__ y, int ldy, const WT* __restrict__ w, float* __restrict__ x,
                                                       int ldx, bf16_t* __restrict__ rounded, int ldr, int dim, float eps,
                                                       const int32_t* __restrict__ place, const float* __restrict__ wts, int top,
                                                       float scale) {
  __shared__ float part[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* yr = y + (size_t)row * ldy;
  auto value = [&](int e) -> float {
    if (place == nullptr) return yr[e];
    float acc = 0.0f;
    for (int j = 0; j < top; ++j) acc = fmaf(wts[(size_t)row * top + j], y[(size_t)place[(size_t)row * top + j] * ldy + e], acc);
    return acc;
  };
  constexpr int MAXV = 8;                       // rows of up to 256 * MAXV elements keep their values in registers
  float v[MAXV];
  float acc = 0.0f;
  if (dim <= 256 * MAXV) {
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int e = tid + 256 * j;
      v[j] = e < dim ? value(e) : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < MAXV; ++j) acc = fmaf(v[j], v[j], acc);
  } else {
    for (int e = tid; e < dim; e += 256) {
      const float ye = value(e);
      acc = fmaf(ye, ye, acc);
    }
  }
  acc = wave_sum(acc);
  if ((tid & 63) == 0) part[tid >> 6] = acc;
  __syncthreads();
  const float total = ((part[0] + part[1]) + part[2]) + part[3];
  const float inv = 1.0f / sqrtf(total / (float)dim + eps);
  float* xr = x + (size_t)row * ldx;
  if (dim <= 256 * MAXV) {
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int e = tid + 256 * j;
      if (e < dim) {
        const float normed = (v[j] * inv) * gm_load(w + e);
        const float nx = scale == 1.0f ? xr[e] + normed : fmaf(scale, normed, xr[e]);
        xr[e] = nx;
        if (rounded != nullptr) rounded[(size_t)row * ldr + e] = f32_to_bf16(nx);
      }
    }
  } else {
    for (int e = tid; e < dim; e += 256) {
      const float normed = (value(e) * inv) * gm_load(w + e);
      const float nx = scale == 1.0f ? xr[e] + normed : fmaf(scale, normed, xr[e]);
      xr[e] = nx;
      if (rounded != nullptr) rounded[(size_t)row * ldr + e] = f32_to_bf16(nx);
    }
  }
}

extern "C" int bw_norm_add(const float* y, int ldy, const void* w, int w_is_bf16, float* x, int ldx, void* rounded, int ldr,
                           int rows, int dim, float eps, const int32_t* place, const float* wts, int top, float scale, void* stream) {
  if (rows <= 0) return 0;
  const dim3 grid(rows);
  if (w_is_bf16)
    hipLaunchKernelGGL(norm_add_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, y, ldy, (const bf16_t*)w, x, ldx, (bf16_t*)rounded, ldr, dim, eps, place, wts, top, scale);
  else
    hipLaunchKernelGGL(norm_add_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, y, ldy, (const float*)w, x, ldx, (bf16_t*)rounded, ldr, dim, eps, place, wts, top, scale);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ the mean of normed branches

// out[r] = (1/n) sum_b (y_b[r] / sqrt(mean(y_b[r]^2) + eps)) * w_b, b ascending: what mixers that run side by side leave,
// each normed over the model width with a weight of its own.  A workgroup a row, the sums of squares as in norm_add_kernel.
struct NormMeanArgs {
  const float* y[4];
  const float* w[4];
  int ldy[4];
  int n;
  float* out;
  int ldo, dim;
  float eps;
};

template <int N>
__global__ __launch_bounds__(256) void norm_mean_kernel(NormMeanArgs a) {
  __shared__ float part[N][4];
  const int row = blockIdx.x, tid = threadIdx.x;
#pragma unroll
  for (int b = 0; b < N; ++b) {
    const float* yr = a.y[b] + (size_t)row * a.ldy[b];
    float acc = 0.0f;
    for (int e = tid; e < a.dim; e += 256) acc = fmaf(yr[e], yr[e], acc);
    acc = wave_sum(acc);
    if ((tid & 63) == 0) part[b][tid >> 6] = acc;
  }
  __syncthreads();
  float inv[N];
#pragma unroll
  for (int b = 0; b < N; ++b)
    inv[b] = 1.0f / sqrtf((((part[b][0] + part[b][1]) + part[b][2]) + part[b][3]) / (float)a.dim + a.eps);
  const float share = 1.0f / (float)N;
  for (int e = tid; e < a.dim; e += 256) {
    float sum = 0.0f;
#pragma unroll
    for (int b = 0; b < N; ++b) sum += (a.y[b][(size_t)row * a.ldy[b] + e] * inv[b]) * a.w[b][e];
    a.out[(size_t)row * a.ldo + e] = sum * share;
  }
}

// x[r] += scale * (z / sqrt(mean(z^2) + eps2) * w2) with z the mean of the normed branches as above: the norm behind the
// mixer rides in the same launch.  Rows of up to 2,048 elements, whose values stay in registers; the bits of
// norm_mean_kernel followed by norm_add_kernel.
template <int N>
__global__ __launch_bounds__(256) void norm_mean_add_kernel(NormMeanArgs a, const float* __restrict__ w2, float eps2, float scale,
                                                            float* __restrict__ x, int ldx) {
  __shared__ float part[N][4];
  __shared__ float part2[4];
  constexpr int MAXV = 8;
  const int row = blockIdx.x, tid = threadIdx.x;
  float v[N][MAXV], wb[N][MAXV], xo[MAXV], wp[MAXV];
  // everything the row needs is asked for before anything is used
#pragma unroll
  for (int j = 0; j < MAXV; ++j) {
    const int e = min(tid + 256 * j, a.dim - 1);
#pragma unroll
    for (int b = 0; b < N; ++b) {
      v[b][j] = a.y[b][(size_t)row * a.ldy[b] + e];
      wb[b][j] = a.w[b][e];
    }
    xo[j] = x[(size_t)row * ldx + e];
    wp[j] = w2[e];
  }
#pragma unroll
  for (int b = 0; b < N; ++b) {
    // (the order of norm_mean_kernel: a thread's elements ascending in one chain)
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j)
      if (tid + 256 * j < a.dim) acc = fmaf(v[b][j], v[b][j], acc);
    acc = wave_sum(acc);
    if ((tid & 63) == 0) part[b][tid >> 6] = acc;
  }
  __syncthreads();
  float inv[N];
#pragma unroll
  for (int b = 0; b < N; ++b)
    inv[b] = 1.0f / sqrtf((((part[b][0] + part[b][1]) + part[b][2]) + part[b][3]) / (float)a.dim + a.eps);
  const float share = 1.0f / (float)N;
  float z[MAXV];
  float acc = 0.0f;
#pragma unroll
  for (int j = 0; j < MAXV; ++j) {
    float sum = 0.0f;
#pragma unroll
    for (int b = 0; b < N; ++b) sum += (v[b][j] * inv[b]) * wb[b][j];
    z[j] = tid + 256 * j < a.dim ? sum * share : 0.0f;
  }
#pragma unroll
  for (int j = 0; j < MAXV; ++j) acc = fmaf(z[j], z[j], acc);
  acc = wave_sum(acc);
  if ((tid & 63) == 0) part2[tid >> 6] = acc;
  __syncthreads();
  const float inv2 = 1.0f / sqrtf((((part2[0] + part2[1]) + part2[2]) + part2[3]) / (float)a.dim + eps2);
  float* xr = x + (size_t)row * ldx;
#pragma unroll
  for (int j = 0; j < MAXV; ++j) {
    const int e = tid + 256 * j;
    if (e < a.dim) {
      const float normed = (z[j] * inv2) * wp[j];
      xr[e] = scale == 1.0f ? xo[j] + normed : fmaf(scale, normed, xo[j]);
    }
  }
}

extern "C" int bw_norm_mean_add(const float* const* y, const int* ldy, const float* const* w, int n, float eps, const float* w2,
                                float eps2, float scale, float* x, int ldx, int rows, int dim, void* stream) {
  if (rows <= 0) return 0;
  if (n < 1 || n > 4 || dim <= 0 || dim > 2048 || ldx < dim || w2 == nullptr) return -2;
  NormMeanArgs a{};
  for (int b = 0; b < n; ++b) {
    if (y[b] == nullptr || w[b] == nullptr || ldy[b] < dim) return -2;
    a.y[b] = y[b];
    a.w[b] = w[b];
    a.ldy[b] = ldy[b];
  }
  a.n = n;
  a.dim = dim;
  a.eps = eps;
  hipStream_t s = (hipStream_t)stream;
  if (n == 1) hipLaunchKernelGGL(norm_mean_add_kernel<1>, dim3(rows), dim3(256), 0, s, a, w2, eps2, scale, x, ldx);
  else if (n == 2) hipLaunchKernelGGL(norm_mean_add_kernel<2>, dim3(rows), dim3(256), 0, s, a, w2, eps2, scale, x, ldx);
  else if (n == 3) hipLaunchKernelGGL(norm_mean_add_kernel<3>, dim3(rows), dim3(256), 0, s, a, w2, eps2, scale, x, ldx);
  else hipLaunchKernelGGL(norm_mean_add_kernel<4>, dim3(rows), dim3(256), 0, s, a, w2, eps2, scale, x, ldx);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_norm_mean(const float* const* y, const int* ldy, const float* const* w, int n, float* out, int ldo, int rows,
                            int dim, float eps, void* stream) {
  if (rows <= 0) return 0;
  if (n < 1 || n > 4 || dim <= 0 || ldo < dim) return -2;
  NormMeanArgs a{};
  for (int b = 0; b < n; ++b) {
    if (y[b] == nullptr || w[b] == nullptr || ldy[b] < dim) return -2;
    a.y[b] = y[b];
    a.w[b] = w[b];
    a.ldy[b] = ldy[b];
  }
  a.n = n;
  a.out = out;
  a.ldo = ldo;
  a.dim = dim;
  a.eps = eps;
  hipStream_t s = (hipStream_t)stream;
  if (n == 1) hipLaunchKernelGGL(norm_mean_kernel<1>, dim3(rows), dim3(256), 0, s, a);
  else if (n == 2) hipLaunchKernelGGL(norm_mean_kernel<2>, dim3(rows), dim3(256), 0, s, a);
  else if (n == 3) hipLaunchKernelGGL(norm_mean_kernel<3>, dim3(rows), dim3(256), 0, s, a);
  else hipLaunchKernelGGL(norm_mean_kernel<4>, dim3(rows), dim3(256), 0, s, a);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ soft cap

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, int ld, int cols, float cap) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= cols) return;
  float* p = x + (size_t)blockIdx.y * ld + e;
  *p = cap * tanhf(*p / cap);
}

__global__ __launch_bounds__(256) void scale_rows_kernel(float* __restrict__ x, int ld, int rows, int cols, float factor) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= cols) return;
  for (int r = blockIdx.y; r < rows; r += gridDim.y) x[(size_t)r * ld + e] *= factor;
}

extern "C" int bw_scale_rows(float* x, int ld, int rows, int cols, float factor, void* stream) {
  if (rows <= 0 || cols <= 0) return 0;
  hipLaunchKernelGGL(scale_rows_kernel, dim3((cols + 255) / 256, rows < 65535 ? rows : 65535), dim3(256), 0, (hipStream_t)stream, x, ld,
                     rows, cols, factor);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_softcap(float* x, int ld, int rows, int cols, float cap, void* stream) {
  if (rows <= 0 || cols <= 0) return 0;
  if (!(cap > 0.0f) || rows > 65535) return -2;
  hipLaunchKernelGGL(softcap_kernel, dim3((cols + 255) / 256, rows), dim3(256), 0, (hipStream_t)stream, x, ld, cols, cap);
  return BW_LAUNCH_CHECK();
}
