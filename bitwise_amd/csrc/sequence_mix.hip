// Kernels of mixers that carry a fixed-size state from token to token instead of a paged cache:
// token shift (fused with the RMSNorm in front of it), the linear recurrence with a matrix state per
// head (gated linear attention with a decay per key channel, and the mLSTM with scalar gates, a
// normaliser and a running maximum), the per-head RMS norm with an output gate behind it, and the
// gated unit of a feed-forward with a choice of activation.
//
// Everything here is 32-bit arithmetic whatever the mode: the state, the gates, their logarithms and
// exponentials, the norms.  The mode only decides the dtype of what is handed to the next matrix product.
//
// A step's rows of one request are consecutive and in position order; ``seq_rows`` holds for every
// request of the step (first row, number of rows) and ``slots`` its state slot.  A request with no rows,
// a negative slot or a negative first position is padding and is skipped: its state is not touched.
#include "common.h"
#include "api.h"

#include <math.h>

namespace {

__device__ __forceinline__ float log_sigmoid(float z) {
  // log(1 / (1 + e^-z)) = min(z, 0) - log1p(e^-|z|)
  return fminf(z, 0.0f) - log1pf(bw_expf(-fabsf(z)));
}

template <typename OT>
__device__ __forceinline__ void store_act(OT* p, float v) {
  if constexpr (sizeof(OT) == 2) *p = f32_to_bf16(v);
  else *p = v;
}

// Sum of squares of a row: lane l runs one fused multiply-add chain over elements l, l+64, ... in ascending order,
// the lanes are joined by the butterflies of wave_sum.  The order depends on the width alone.
__device__ __forceinline__ float row_sumsq(const float* __restrict__ xr, int dim, int lane) {
  float acc = 0.0f;
  for (int i = lane; i < dim; i += 64) acc = fmaf(xr[i], xr[i], acc);
  return wave_sum(acc);
}

// ------------------------------------------------------------------------- RMSNorm + token shift

// out[r][m] = h[r] + (h'[r] - h[r]) * mix[m] for each of nmix mixing vectors (out rows hold nmix blocks of dim elements), with
// h = (x * inv_rms) * w and h' the h of the request's previous token: the
// row above, or for the first row of a request in this step what the state slot holds (zeros for a new request).
// The wave of a request's first row also leaves the h of the request's last row in the slot, after it has read it:
// nothing else reads or writes that slot in this launch.  A wave a row.
template <typename OT>
__global__ __launch_bounds__(256) void norm_shift_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w,
                                                         const float* __restrict__ mix, float* __restrict__ state,
                                                         long long state_ld, const int32_t* __restrict__ positions,
                                                         const int32_t* __restrict__ row_seq,
                                                         const int32_t* __restrict__ seq_rows,
                                                         const int32_t* __restrict__ slots, OT* __restrict__ out, int ldo,
                                                         int rows, int dim, float eps, int nmix) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * (blockDim.x >> 6) + wave_index();
  if (row >= rows) return;
  if (positions[row] < 0) return;
  const int seq = row_seq[row];
  const int first = seq_rows[2 * seq], count = seq_rows[2 * seq + 1];
  const int slot = slots[seq];
  if (slot < 0 || count <= 0) return;
  const float* xr = x + (size_t)row * ldx;
  float* st = state + (size_t)slot * state_ld;
  OT* o = out + (size_t)row * ldo;
  if ((dim & 3) == 0 && (ldx & 3) == 0 && (ldo & 3) == 0 && (state_ld & 3) == 0) {
    // rows of whole 16-byte vectors: lane l owns vectors l, l+64, ...; four of them (and of everything that goes with them) are
    // asked for before the first is used
    const int nvec = dim >> 2;
    const bool is_first = row == first;
    const int last = first + count - 1;
    const f32x4* xv = reinterpret_cast<const f32x4*>(xr);
    const f32x4* pv = is_first ? reinterpret_cast<const f32x4*>(st) : reinterpret_cast<const f32x4*>(xr - ldx);
    const f32x4* lv = reinterpret_cast<const f32x4*>(x + (size_t)last * ldx);
    const f32x4* wv = reinterpret_cast<const f32x4*>(w);
    const f32x4* mv = reinterpret_cast<const f32x4*>(mix);
    const float inv = 1.0f / sqrtf(row_sumsq_vec(xv, nvec, lane) / (float)dim + eps);
    const float invp = is_first ? 1.0f : 1.0f / sqrtf(row_sumsq_vec(pv, nvec, lane) / (float)dim + eps);
    const float invl = !is_first || last == row ? inv : 1.0f / sqrtf(row_sumsq_vec(lv, nvec, lane) / (float)dim + eps);
    constexpr int UN = 4;
    for (int c0 = 0; c0 < nvec; c0 += 64 * UN) {
      f32x4 xq[UN], pq[UN], lq[UN], wq[UN], mq[UN];
#pragma unroll
      for (int jj = 0; jj < UN; ++jj) {
        const int c = min(c0 + 64 * jj + lane, nvec - 1);
        xq[jj] = xv[c];
        pq[jj] = pv[c];
        wq[jj] = wv[c];
        mq[jj] = mv[c];
        lq[jj] = is_first ? lv[c] : xq[jj];
      }
#pragma unroll
      for (int jj = 0; jj < UN; ++jj) {
        const int c = c0 + 64 * jj + lane;
        if (c >= nvec) continue;
        f32x4 hq, dq, keep;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          hq[e] = (xq[jj][e] * inv) * wq[jj][e];
          const float hp = is_first ? pq[jj][e] : (pq[jj][e] * invp) * wq[jj][e];
          dq[e] = hp - hq[e];
          keep[e] = (lq[jj][e] * invl) * wq[jj][e];
        }
        // (the further mixing vectors four at a time: their loads are all asked for before the first is used)
        for (int m0 = 0; m0 < nmix; m0 += 4) {
          f32x4 mm[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) mm[k] = m0 + k == 0 ? mq[jj] : mv[(size_t)min(m0 + k, nmix - 1) * nvec + c];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            if (m0 + k >= nmix) continue;
            f32x4 r;
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = fmaf(dq[e], mm[k][e], hq[e]);
            OT* om = o + (size_t)(m0 + k) * dim;
            if constexpr (sizeof(OT) == 2) {
              *reinterpret_cast<u32x2*>(om + 4 * c) = (u32x2){pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3])};
            } else {
              *reinterpret_cast<f32x4*>(om + 4 * c) = r;
            }
          }
        }
        if (is_first) reinterpret_cast<f32x4*>(st)[c] = keep;
      }
    }
    return;
  }
  const float inv = 1.0f / sqrtf(row_sumsq(xr, dim, lane) / (float)dim + eps);
  if (row != first) {
    const float* xp = xr - ldx;
    const float invp = 1.0f / sqrtf(row_sumsq(xp, dim, lane) / (float)dim + eps);
    for (int i = lane; i < dim; i += 64) {
      const float h = (xr[i] * inv) * w[i];
      const float hp = (xp[i] * invp) * w[i];
      for (int m = 0; m < nmix; ++m) store_act(o + (size_t)m * dim + i, fmaf(hp - h, mix[(size_t)m * dim + i], h));
    }
    return;
  }
  const int last = first + count - 1;
  const float* xl = x + (size_t)last * ldx;
  const float invl = last == row ? inv : 1.0f / sqrtf(row_sumsq(xl, dim, lane) / (float)dim + eps);
  for (int i = lane; i < dim; i += 64) {
    const float h = (xr[i] * inv) * w[i];
    const float hp = st[i];
    for (int m = 0; m < nmix; ++m) store_act(o + (size_t)m * dim + i, fmaf(hp - h, mix[(size_t)m * dim + i], h));
    st[i] = (xl[i] * invl) * w[i];
  }
}

// The same for steps of few rows, a workgroup a row: all of a row's operands (the row, the row before or the slot's, the
// request's last row, the weight and up to eight mixing vectors) are asked for at once, the rows pass through LDS, and a
// wave each runs row_sumsq_vec over them from there: the chains, and so the bits, of the kernel above.  Rows of whole
// 16-byte vectors, up to 4,096 elements.
#define SHIFT_ROW_MAXV 4
#define SHIFT_ROW_MAXMIX 8
template <typename OT>
__global__ __launch_bounds__(256) void norm_shift_row_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w,
                                                             const float* __restrict__ mix, float* __restrict__ state,
                                                             long long state_ld, const int32_t* __restrict__ positions,
                                                             const int32_t* __restrict__ row_seq,
                                                             const int32_t* __restrict__ seq_rows,
                                                             const int32_t* __restrict__ slots, OT* __restrict__ out, int ldo,
                                                             int rows, int dim, float eps, int nmix) {
  extern __shared__ float shift_lds[];            // three rows of dim elements, then three numbers
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  if (positions[row] < 0) return;
  const int seq = row_seq[row];
  const int first = seq_rows[2 * seq], count = seq_rows[2 * seq + 1];
  const int slot = slots[seq];
  if (slot < 0 || count <= 0) return;
  const float* xr = x + (size_t)row * ldx;
  float* st = state + (size_t)slot * state_ld;
  OT* o = out + (size_t)row * ldo;
  const int nvec = dim >> 2;
  const bool is_first = row == first;
  const int last = first + count - 1;
  const bool need_p = !is_first, need_l = is_first && last != row;
  const f32x4* xv = reinterpret_cast<const f32x4*>(xr);
  const f32x4* pv = is_first ? reinterpret_cast<const f32x4*>(st) : reinterpret_cast<const f32x4*>(xr - ldx);
  const f32x4* lv = reinterpret_cast<const f32x4*>(x + (size_t)last * ldx);
  const f32x4* wvp = reinterpret_cast<const f32x4*>(w);
  const f32x4* mv = reinterpret_cast<const f32x4*>(mix);
  f32x4* sx = reinterpret_cast<f32x4*>(shift_lds);
  f32x4* sp = sx + nvec;
  f32x4* sl = sp + nvec;
  float* invs = reinterpret_cast<float*>(sl + nvec);
  f32x4 xq[SHIFT_ROW_MAXV], pq[SHIFT_ROW_MAXV], lq[SHIFT_ROW_MAXV], wq[SHIFT_ROW_MAXV], mm[SHIFT_ROW_MAXV][SHIFT_ROW_MAXMIX];
#pragma unroll
  for (int j = 0; j < SHIFT_ROW_MAXV; ++j) {
    const int c = min(tid + 256 * j, nvec - 1);
    xq[j] = xv[c];
    pq[j] = pv[c];
    wq[j] = wvp[c];
    lq[j] = need_l ? lv[c] : xq[j];
#pragma unroll
    for (int m = 0; m < SHIFT_ROW_MAXMIX; ++m) mm[j][m] = mv[(size_t)min(m, nmix - 1) * nvec + c];
  }
#pragma unroll
  for (int j = 0; j < SHIFT_ROW_MAXV; ++j) {
    const int c = tid + 256 * j;
    if (c < nvec) {
      sx[c] = xq[j];
      if (need_p) sp[c] = pq[j];
      if (need_l) sl[c] = lq[j];
    }
  }
  __syncthreads();
  if (wv == 0 || (wv == 1 && need_p) || (wv == 2 && need_l)) {
    const float ss = row_sumsq_vec(wv == 0 ? sx : (wv == 1 ? sp : sl), nvec, lane);
    if (lane == 0) invs[wv] = 1.0f / sqrtf(ss / (float)dim + eps);
  }
  __syncthreads();
  const float inv = invs[0];
  const float invp = need_p ? invs[1] : 1.0f;
  const float invl = need_l ? invs[2] : inv;
#pragma unroll
  for (int j = 0; j < SHIFT_ROW_MAXV; ++j) {
    const int c = tid + 256 * j;
    if (c >= nvec) continue;
    f32x4 hq, dq, keep;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      hq[e] = (xq[j][e] * inv) * wq[j][e];
      const float hp = is_first ? pq[j][e] : (pq[j][e] * invp) * wq[j][e];
      dq[e] = hp - hq[e];
      keep[e] = (lq[j][e] * invl) * wq[j][e];
    }
#pragma unroll
    for (int m = 0; m < SHIFT_ROW_MAXMIX; ++m) {
      if (m >= nmix) continue;
      f32x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = fmaf(dq[e], mm[j][m][e], hq[e]);
      OT* om = o + (size_t)m * dim;
      if constexpr (sizeof(OT) == 2) {
        *reinterpret_cast<u32x2*>(om + 4 * c) = (u32x2){pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3])};
      } else {
        *reinterpret_cast<f32x4*>(om + 4 * c) = r;
      }
    }
    if (is_first) reinterpret_cast<f32x4*>(st)[c] = keep;
  }
}

// ------------------------------------------------------------------------- the linear recurrence

enum { RECUR_DECAY_PER_CHANNEL = 0, RECUR_SCALAR_GATES = 1, RECUR_BONUS_DECAY = 2, RECUR_FIXED_DECAY = 3 };

// The sum over the lanes l, l + 64/SPLIT, ... that hold the parts of one column (every one of them gets it).
template <int SPLIT>
__device__ __forceinline__ float join_parts(float v) {
  if constexpr (SPLIT >= 2) {
    float lower, upper;
    lane_halves<32>(v, lower, upper);
    v = lower + upper;
    if constexpr (SPLIT == 4) {
      lane_halves<16>(v, lower, upper);
      v = lower + upper;
    }
  }
  return v;
}

struct RecurArgs {
  const float* proj;       // [rows, ldp]: the rows' stacked projections
  int ldp, q_off, k_off, v_off;
  const float* gate;       // per channel: decay logits [rows, ldg] at gate_off + head*dim + d;
  int ldg, gate_off, gate2_off;   // scalar gates: input gate at gate_off + head, forget gate at gate2_off + head
  const float* bias;       // per channel: [heads*dim]; scalar gates: input-gate bias [heads]
  const float* bias2;      // scalar gates: forget-gate bias [heads]
  float param;             // per channel: 1 / tau; scalar gates: the cap
  float qscale, kscale;
  float* state;            // [slots, state_ld]: S [heads][dim][vdim]; scalar gates also n [heads][dim] and m [heads]
  long long state_ld;
  float* out;              // [rows, ldo]: head h at columns h*vdim ..
  int ldo;
  const int32_t* seq_rows;
  const int32_t* slots;
  const int32_t* positions;
  int heads, dim, vdim;
  // long prompt portions in three passes (PHASE 1 to 3): chunks [n][4] = (first row, rows, request of the step, 1 if it is
  // the request's last chunk); records of heads x (dim*vdim + dim + 2) floats per chunk: S, a vector, two scalars
  const int32_t* chunks;
  float* local;            // per chunk, from zero state: S, and the decay over the chunk (per channel: the product of the
                           // decays; scalar gates: n, the maximum from -inf, the sum of the log forget gates)
  float* start;            // per chunk: the state it starts from (S; scalar gates: n, m)
};

// One wave per (request, head, block of 64, 32 or 16 value columns: see SPLIT).  Lane j keeps column j of the head's state matrix in
// registers (one element per key channel), so the read-out S^T q needs no exchange between lanes; the tokens' q, k and
// decays come through LDS in chunks of RC tokens and are read from there by all lanes at once.
//
// RECUR_DECAY_PER_CHANNEL:  S[d][j] <- alpha[d] S[d][j] + k[d] v[j],  alpha = exp(logsigmoid(z + bias) / tau);  o[j] = sum_d S[d][j] q[d].
// RECUR_SCALAR_GATES:  i = cap tanh((gi + bi) / cap), f = logsigmoid(cap tanh((gf + bf) / cap)), m' = max(f + m, i),
//   S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise with k alone, o[j] = (S^T q)[j] / (max(|n.q|, e^-m') + 1e-6).
//   n is spread over the lanes (lane l holds n[l], n[l+64], ...); every wave of a head computes it, the wave of
//   column block 0 stores it.
//
// RECUR_BONUS_DECAY:  alpha[d] = exp(-exp(z[d] + bias[d]));  o[j] = sum_d (S[d][j] + u[d] k[d] v[j]) q[d] with the S of the token
//   before (the token's own k v^T is read through the bonus u = bias2 [heads*dim]), then S[d][j] <- alpha[d] S[d][j] + k[d] v[j].
// RECUR_FIXED_DECAY:  as per channel with one constant decay a head, alpha[d] = bias[head]; no logits are read.
// (q is multiplied by qscale and k by kscale on their way into LDS.)
//
// A request's long portion can also run in three passes over chunks of its rows, which gives every chunk waves of its
// own: PHASE 1 runs every chunk from a zero state (no read-out) and leaves the chunk's own contribution and its decay;
// recurrence_scan_kernel walks a request's chunks in order and leaves the state each one starts from; PHASE 3 runs every
// chunk from there with the read-out, and the request's last chunk leaves the state in the slot.  PHASE 0 is the whole
// portion by one wave.  The passes differ from PHASE 0 by the rounding of the scan's sums only.
#define RC 16
#define RW 4             // waves of a workgroup: neighbouring column blocks of one head, which share the staged tokens
template <int MODE, int DPAD, int PHASE>
__global__ __launch_bounds__(64 * RW) void linear_recurrence_kernel(RecurArgs a) {
  constexpr bool GATES = MODE == RECUR_SCALAR_GATES;
  constexpr bool BONUS = MODE == RECUR_BONUS_DECAY, FIXED = MODE == RECUR_FIXED_DECAY;
  constexpr int NN = (DPAD + 63) / 64;
  constexpr bool READ_OUT = PHASE != 1;
  // A column's key channels are split over SPLIT lanes (lane l, l + COLS, ... hold consecutive parts of column l mod COLS): a
  // lane's part of the state is at most 64 registers and a token costs a lane DPAD / SPLIT steps, so a head has more and
  // shorter waves.  The parts' read-outs are added by the swaps of the wave's halves and quarters, in one order whatever
  // runs the head (a single token, a portion, a chunk): the split depends on the head's size alone.
  constexpr int SPLIT = DPAD >= 64 ? 4 : (DPAD >= 32 ? 2 : 1);
  constexpr int DH = DPAD / SPLIT, COLS = 64 / SPLIT;
  __shared__ float qs[RC][DPAD];
  __shared__ float ks[RC][DPAD];
  __shared__ float as[GATES ? 1 : RC][GATES ? 1 : DPAD];
  __shared__ float gi[RC], gf[RC];
  __shared__ float vs[RW][RC][64];
  __shared__ float us[BONUS ? DPAD : 1];
  const int lane = threadIdx.x & 63, wv = wave_index();
  const int cb = blockIdx.x * RW + wv, h = blockIdx.y;
  const int dim = a.dim, vdim = a.vdim;
  const size_t rec = (size_t)dim * vdim + dim + 2;
  int first, count, slot;
  bool leaves_state = true;
  if constexpr (PHASE == 0) {
    const int s = blockIdx.z;
    first = a.seq_rows[2 * s];
    count = a.seq_rows[2 * s + 1];
    slot = a.slots[s];
  } else {
    const int c = blockIdx.z;
    first = a.chunks[4 * c];
    count = a.chunks[4 * c + 1];
    slot = a.slots[a.chunks[4 * c + 2]];
    leaves_state = a.chunks[4 * c + 3] != 0;
  }
  if (count <= 0 || slot < 0) return;
  if (a.positions[first] < 0) return;
  const int col = lane % COLS, dbase = (lane / COLS) * DH;
  const int j = cb * COLS + col;
  const bool live = j < vdim;
  float* st = a.state + (size_t)slot * a.state_ld;
  float* S = st + (size_t)h * dim * vdim;
  float* nv = st + (size_t)a.heads * dim * vdim + (size_t)h * dim;
  float* mv = st + (size_t)a.heads * dim * vdim + (size_t)a.heads * dim + h;
  // where this wave's state comes from: the slot, nothing, or the chunk's start record
  const float* S_in = S;
  const float* nv_in = nv;
  const float* mv_in = mv;
  if constexpr (PHASE == 3) {
    S_in = a.start + ((size_t)blockIdx.z * a.heads + h) * rec;
    nv_in = S_in + (size_t)dim * vdim;
    mv_in = nv_in + dim;
  }

  float Sreg[DH];
#pragma unroll
  for (int d = 0; d < DH; ++d) Sreg[d] = (PHASE != 1 && live && dbase + d < dim) ? S_in[(size_t)(dbase + d) * vdim + j] : 0.0f;
  float nreg[NN];          // scalar gates: the normaliser; per channel in PHASE 1: the product of the chunk's decays
  float m = 0.0f, fsum = 0.0f;
  if constexpr (GATES) {
#pragma unroll
    for (int i = 0; i < NN; ++i) nreg[i] = (PHASE != 1 && lane + 64 * i < dim) ? nv_in[lane + 64 * i] : 0.0f;
    m = PHASE == 1 ? -INFINITY : *mv_in;
  } else {
#pragma unroll
    for (int i = 0; i < NN; ++i) nreg[i] = 1.0f;
  }

  if constexpr (BONUS) {
    for (int d = threadIdx.x; d < DPAD; d += 64 * RW) us[d] = d < dim ? a.bias2[h * dim + d] : 0.0f;
  }
  const float fixed_decay = FIXED ? a.bias[h] : 0.0f;
  for (int t0 = 0; t0 < count; t0 += RC) {
    const int tc = min(RC, count - t0);
    __syncthreads();
    // eight elements a lane at a time: their loads are all asked for before the first is used
    for (int e0 = 0; e0 < tc * DPAD; e0 += 64 * RW * 8) {
      float qv[8], kv[8], zv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int e = e0 + 64 * RW * u + (int)threadIdx.x;
        const int t = e / DPAD, d = e % DPAD;
        const bool in = e < tc * DPAD && d < dim;
        const size_t row = (size_t)(first + t0 + min(t, tc - 1));
        const float* pr = a.proj + row * a.ldp;
        qv[u] = in ? pr[a.q_off + h * dim + d] : 0.0f;
        kv[u] = in ? pr[a.k_off + h * dim + d] : 0.0f;
        if constexpr (!GATES && !FIXED) zv[u] = in ? a.gate[row * a.ldg + a.gate_off + h * dim + d] + a.bias[h * dim + d] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int e = e0 + 64 * RW * u + (int)threadIdx.x;
        if (e >= tc * DPAD) continue;
        const int t = e / DPAD, d = e % DPAD;
        qs[t][d] = qv[u] * a.qscale;
        ks[t][d] = kv[u] * a.kscale;
        if constexpr (FIXED) as[t][d] = d < dim ? fixed_decay : 0.0f;
        else if constexpr (BONUS) as[t][d] = d < dim ? bw_expf(-bw_expf(zv[u])) : 0.0f;
        else if constexpr (!GATES) as[t][d] = d < dim ? bw_expf(log_sigmoid(zv[u]) * a.param) : 0.0f;
      }
    }
    if constexpr (GATES) {
      if (wv == 0 && lane < tc) {
        const float* pr = a.proj + (size_t)(first + t0 + lane) * a.ldp;
        const float cap = a.param;
        gi[lane] = cap * tanhf((pr[a.gate_off + h] + a.bias[h]) / cap);
        gf[lane] = log_sigmoid(cap * tanhf((pr[a.gate2_off + h] + a.bias2[h]) / cap));
      }
    }
    // (a column's lanes read what its first lane wrote)
    if (lane < COLS) {
#pragma unroll
      for (int t = 0; t < RC; ++t)
        vs[wv][t][col] = (live && t < tc) ? a.proj[(size_t)(first + t0 + t) * a.ldp + a.v_off + h * vdim + j] : 0.0f;
    }
    __syncthreads();
    for (int t = 0; t < tc; ++t) {
      float o = 0.0f;
      if constexpr (!GATES) {
        const float v = vs[wv][t][col];
#pragma unroll
        for (int d = 0; d < DH; ++d) {
          if constexpr (BONUS) {
            const float kv = ks[t][dbase + d] * v;
            if constexpr (READ_OUT) o = fmaf(fmaf(us[dbase + d], kv, Sreg[d]), qs[t][dbase + d], o);
            Sreg[d] = fmaf(as[t][dbase + d], Sreg[d], kv);
          } else {
            Sreg[d] = fmaf(as[t][dbase + d], Sreg[d], ks[t][dbase + d] * v);
            if constexpr (READ_OUT) o = fmaf(Sreg[d], qs[t][dbase + d], o);
          }
        }
        if constexpr (PHASE == 1) {
#pragma unroll
          for (int i = 0; i < NN; ++i)
            if (lane + 64 * i < DPAD) nreg[i] *= as[t][lane + 64 * i];
        }
      } else {
        const float ig = gi[t], fg = gf[t];
        const float mn = fmaxf(fg + m, ig);
        const float fa = bw_expf(fg + m - mn);
        const float ib = bw_expf(ig - mn);
        m = mn;
        fsum += fg;
        const float bv = ib * vs[wv][t][col];
#pragma unroll
        for (int d = 0; d < DH; ++d) {
          Sreg[d] = fmaf(fa, Sreg[d], ks[t][dbase + d] * bv);
          if constexpr (READ_OUT) o = fmaf(Sreg[d], qs[t][dbase + d], o);
        }
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < NN; ++i) {
          const int d = lane + 64 * i;
          if (d < DPAD) {
            nreg[i] = fmaf(fa, nreg[i], ib * ks[t][d]);
            part = fmaf(nreg[i], qs[t][d], part);
          }
        }
        if constexpr (READ_OUT) {
          o = join_parts<SPLIT>(o);
          const float nq = wave_sum(part);
          o = o / (fmaxf(fabsf(nq), bw_expf(-mn)) + 1e-6f);
        }
      }
      if constexpr (READ_OUT) {
        if constexpr (!GATES) o = join_parts<SPLIT>(o);
        if (live && lane < COLS) a.out[(size_t)(first + t0 + t) * a.ldo + h * vdim + j] = o;
      }
    }
  }
  // where the state goes: the slot (PHASE 3: from the request's last chunk only), or the chunk's own record
  float* S_out = S;
  float* nv_out = nv;
  float* mv_out = mv;
  if constexpr (PHASE == 1) {
    S_out = a.local + ((size_t)blockIdx.z * a.heads + h) * rec;
    nv_out = S_out + (size_t)dim * vdim;
    mv_out = nv_out + dim;
  }
  if (PHASE == 3 && !leaves_state) return;
  if (live) {
#pragma unroll
    for (int d = 0; d < DH; ++d)
      if (dbase + d < dim) S_out[(size_t)(dbase + d) * vdim + j] = Sreg[d];
  }
  if (cb == 0 && (GATES || PHASE == 1)) {
#pragma unroll
    for (int i = 0; i < NN; ++i)
      if (lane + 64 * i < dim) nv_out[lane + 64 * i] = nreg[i];
    if (GATES && lane == 0) {
      mv_out[0] = m;
      if (PHASE == 1) mv_out[1] = fsum;
    }
  }
}

// A request's chunks in order: the state each one starts from, out of the slot's state and the chunks' own contributions
// and decays.  A thread per element of a head's record; every thread of a head walks the same scalars.
//   per channel:   S' = decay[d] * S + S_local
//   scalar gates:  m' = max(F + m, b), S' = e^(F + m - m') S + e^(b - m') S_local, n likewise (F: the chunk's sum of log
//                  forget gates, b: its maximum from -inf)
template <int MODE>
__global__ __launch_bounds__(256) void recurrence_scan_kernel(RecurArgs a, const int32_t* __restrict__ spans) {
  constexpr bool GATES = MODE == RECUR_SCALAR_GATES;
  const int dim = a.dim, vdim = a.vdim, h = blockIdx.y;
  const int seq = spans[3 * blockIdx.z], c0 = spans[3 * blockIdx.z + 1], nc = spans[3 * blockIdx.z + 2];
  const int slot = a.slots[seq];
  if (slot < 0 || nc <= 0) return;
  const size_t rec = (size_t)dim * vdim + dim + 2;
  const int e = blockIdx.x * 256 + threadIdx.x;
  const int sd = dim * vdim;
  const int mine = GATES ? sd + dim + 1 : sd;          // elements a head has to carry: S, and with scalar gates n and m
  if (e >= mine) return;
  const float* st = a.state + (size_t)slot * a.state_ld;
  float val, m = 0.0f;
  if (e < sd) val = st[(size_t)h * sd + e];
  else if (e < sd + dim) val = st[(size_t)a.heads * sd + (size_t)h * dim + (e - sd)];
  else val = 0.0f;
  if constexpr (GATES) m = st[(size_t)a.heads * sd + (size_t)a.heads * dim + h];
  for (int c = c0; c < c0 + nc; ++c) {
    const float* loc = a.local + ((size_t)c * a.heads + h) * rec;
    float* out = a.start + ((size_t)c * a.heads + h) * rec;
    if constexpr (GATES) {
      out[e] = e == sd + dim ? m : val;
      const float b = loc[sd + dim], F = loc[sd + dim + 1];
      const float mn = fmaxf(F + m, b);
      const float ca = bw_expf(F + m - mn), cl = bw_expf(b - mn);
      if (e < sd + dim) val = fmaf(ca, val, cl * loc[e]);
      m = mn;
    } else {
      out[e] = val;
      val = fmaf(loc[sd + e / vdim], val, loc[e]);
    }
  }
}

template <int MODE, int PHASE>
int launch_recurrence(const RecurArgs& a, int units, hipStream_t s) {
  const int cols = a.dim > 32 ? 16 : (a.dim > 16 ? 32 : 64);      // (columns a wave: linear_recurrence_kernel's COLS)
  const dim3 grid((a.vdim + RW * cols - 1) / (RW * cols), a.heads, units), block(64 * RW);
  if (a.dim <= 16) hipLaunchKernelGGL((linear_recurrence_kernel<MODE, 16, PHASE>), grid, block, 0, s, a);
  else if (a.dim <= 32) hipLaunchKernelGGL((linear_recurrence_kernel<MODE, 32, PHASE>), grid, block, 0, s, a);
  else if (a.dim <= 64) hipLaunchKernelGGL((linear_recurrence_kernel<MODE, 64, PHASE>), grid, block, 0, s, a);
  else if (a.dim <= 128) hipLaunchKernelGGL((linear_recurrence_kernel<MODE, 128, PHASE>), grid, block, 0, s, a);
  else if (a.dim <= 256) hipLaunchKernelGGL((linear_recurrence_kernel<MODE, 256, PHASE>), grid, block, 0, s, a);
  else return -4;
  return BW_LAUNCH_CHECK();
}

template <int MODE>
int launch_recurrence_passes(const RecurArgs& a, int nseq, int nchunks, const int32_t* spans, int nspans, hipStream_t s) {
  int rc = 0;
  if (nseq > 0) rc = launch_recurrence<MODE, 0>(a, nseq, s);
  if (rc != 0 || nchunks <= 0) return rc;
  rc = launch_recurrence<MODE, 1>(a, nchunks, s);
  if (rc != 0) return rc;
  const int mine = a.dim * a.vdim + (MODE == RECUR_SCALAR_GATES ? a.dim + 1 : 0);
  hipLaunchKernelGGL(recurrence_scan_kernel<MODE>, dim3((mine + 255) / 256, a.heads, nspans), dim3(256), 0, s, a, spans);
  rc = BW_LAUNCH_CHECK();
  if (rc != 0) return rc;
  return launch_recurrence<MODE, 3>(a, nchunks, s);
}

// ------------------------------------------------------------------------- per-head RMS norm and output gate

enum { GATE_SIGMOID = 0, GATE_SILU = 1 };

// out[r][h*vdim + j] = o[r][h][j] / sqrt(mean_j o^2 + eps) * weight[h*wstride + j] * gate(g[r][h*vdim + j]); a wave per (row, head).
template <typename OT>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, int ldi, const float* __restrict__ weight,
                                                             int wstride, const float* __restrict__ g, int ldg, int gate,
                                                             OT* __restrict__ out, int ldo, const int32_t* __restrict__ positions,
                                                             int rows, int heads, int vdim, float eps) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * (blockDim.x >> 6) + wave_index();
  if (item >= rows * heads) return;
  const int row = item / heads, h = item % heads;
  if (positions[row] < 0) return;
  const float* orow = o + (size_t)row * ldi + h * vdim;
  const float inv = 1.0f / sqrtf(row_sumsq(orow, vdim, lane) / (float)vdim + eps);
  const float* grow = g + (size_t)row * ldg + h * vdim;
  const float* wr = weight + (size_t)h * wstride;
  OT* dst = out + (size_t)row * ldo + h * vdim;
  for (int jj = lane; jj < vdim; jj += 64) {
    const float z = grow[jj];
    const float sg = 1.0f / (1.0f + bw_expf(-z));
    const float gv = gate == GATE_SILU ? z * sg : sg;
    store_act(dst + jj, ((orow[jj] * inv) * wr[jj]) * gv);
  }
}

// ------------------------------------------------------------------------- gated unit

enum { ACT_SILU = 0, ACT_GELU_TANH = 1, ACT_CLAMPED_SWISH = 2 };

template <typename OT>
__global__ void glu_kernel(const float* __restrict__ gu, int ldg, OT* __restrict__ hout, long long n, int inter, int act, float limit,
                           float alpha, const float* __restrict__ row_gate, int ld_row_gate) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const long long row = idx / inter;
  const int c = (int)(idx % inter);
  float g = gu[row * ldg + c], u = gu[row * ldg + inter + c];
  float h;
  if (act == ACT_GELU_TANH) {
    const float inner = 0.7978845608028654f * (g + 0.044715f * ((g * g) * g));
    h = ((0.5f * g) * (1.0f + tanhf(inner))) * u;
  } else if (act == ACT_CLAMPED_SWISH) {
    h = clamped_swish_times<sizeof(OT) == 2>(g, u, limit, alpha);
  } else {
    h = (g * (1.0f / (1.0f + bw_expf(-g)))) * u;
  }
  if (row_gate != nullptr) h *= 1.0f / (1.0f + bw_expf(-row_gate[row * ld_row_gate]));
  store_act(hout + idx, h);
}


// ------------------------------------------------------------------------- rotation of 32-bit projections in place

// Sections of a row of 32-bit projections ([heads][dim] each, at columns off[s]) turned in place by the row's position:
// of every head's first rot elements, element i < rot/2 is paired with element i + rot/2, (u, v) -> (u c - v s, v c + u s)
// with c, s from the tables' row of the position.  A thread a pair.
struct RotateRowsArgs {
  float* x;
  int ldx, rows, heads, dim, rot, sections;
  int off[2];
  const float* cos_table;     // [positions, rot / 2]
  const float* sin_table;
  const int32_t* positions;
};

__global__ __launch_bounds__(256) void rotate_halves_rows_kernel(RotateRowsArgs a) {
  const int half = a.rot / 2;
  const int per_row = a.sections * a.heads * half;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)a.rows * per_row) return;
  const int row = (int)(idx / per_row);
  int r = (int)(idx % per_row);
  const int sec = r / (a.heads * half);
  r %= a.heads * half;
  const int h = r / half, i = r % half;
  const int pos = a.positions[row];
  if (pos < 0) return;
  float* p = a.x + (size_t)row * a.ldx + a.off[sec] + (size_t)h * a.dim;
  const float c = a.cos_table[(size_t)pos * half + i], s = a.sin_table[(size_t)pos * half + i];
  const float u = p[i], v = p[i + half];
  p[i] = u * c - v * s;
  p[i + half] = v * c + u * s;
}

// x <- tanh(x) over [rows, cols] of 32-bit values
__global__ __launch_bounds__(256) void tanh_rows_kernel(float* __restrict__ x, int ld, int rows, int cols) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)rows * cols) return;
  float* p = x + (idx / cols) * ld + (idx % cols);
  *p = tanhf(*p);
}

}  // namespace

extern "C" int bw_norm_shift(const float* x, int ldx, const float* w, const float* mix, float* state, long long state_ld,
                             const int32_t* positions, const int32_t* row_seq, const int32_t* seq_rows,
                             const int32_t* slots, void* out, int out_is_bf16, int ldo, int rows, int dim, float eps,
                             int nmix, void* stream) {
  if (rows <= 0) return 0;
  if (dim <= 0 || nmix < 1 || ldx < dim || (long long)ldo < (long long)nmix * dim || state_ld < dim) return -2;
  hipStream_t s = (hipStream_t)stream;
  if (rows <= 64 && (dim & 3) == 0 && (ldx & 3) == 0 && (ldo & 3) == 0 && (state_ld & 3) == 0 && dim <= 1024 * SHIFT_ROW_MAXV &&
      nmix <= SHIFT_ROW_MAXMIX) {
    const size_t bytes = (size_t)(3 * dim + 4) * sizeof(float);
    if (out_is_bf16)
      hipLaunchKernelGGL(norm_shift_row_kernel<bf16_t>, dim3(rows), dim3(256), bytes, s, x, ldx, w, mix, state, state_ld, positions,
                         row_seq, seq_rows, slots, (bf16_t*)out, ldo, rows, dim, eps, nmix);
    else
      hipLaunchKernelGGL(norm_shift_row_kernel<float>, dim3(rows), dim3(256), bytes, s, x, ldx, w, mix, state, state_ld, positions,
                         row_seq, seq_rows, slots, (float*)out, ldo, rows, dim, eps, nmix);
    return BW_LAUNCH_CHECK();
  }
  const dim3 grid((rows + 3) / 4), block(256);
  if (out_is_bf16)
    hipLaunchKernelGGL(norm_shift_kernel<bf16_t>, grid, block, 0, s, x, ldx, w, mix, state, state_ld, positions, row_seq,
                       seq_rows, slots, (bf16_t*)out, ldo, rows, dim, eps, nmix);
  else
    hipLaunchKernelGGL(norm_shift_kernel<float>, grid, block, 0, s, x, ldx, w, mix, state, state_ld, positions, row_seq,
                       seq_rows, slots, (float*)out, ldo, rows, dim, eps, nmix);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_linear_recurrence(int mode, const float* proj, int ldp, int q_off, int k_off, int v_off, const float* gate,
                                    int ldg, int gate_off, int gate2_off, const float* bias, const float* bias2, float param,
                                    float qscale, float kscale, float* state, long long state_ld, float* out, int ldo,
                                    const int32_t* seq_rows, const int32_t* slots, const int32_t* positions, int nseq,
                                    int heads, int dim, int vdim, const int32_t* chunks, int nchunks, const int32_t* spans,
                                    int nspans, float* scan_local, float* scan_start, long long scan_floats, void* stream) {
  if (nseq <= 0 && nchunks <= 0) return 0;
  if (nchunks > 0) {
    if (chunks == nullptr || spans == nullptr || nspans <= 0 || scan_local == nullptr || scan_start == nullptr) return -2;
    if (scan_floats < (long long)nchunks * heads * ((long long)dim * vdim + dim + 2)) return -6;
  }
  if (heads <= 0 || dim <= 0 || vdim <= 0 || ldo < heads * vdim) return -2;
  const long long need = (long long)heads * dim * vdim + (mode == RECUR_SCALAR_GATES ? (long long)heads * dim + heads : 0);
  if (state_ld < need) return -2;
  if (bias == nullptr || (mode != RECUR_FIXED_DECAY && gate == nullptr) || ((mode == RECUR_SCALAR_GATES || mode == RECUR_BONUS_DECAY) && bias2 == nullptr))
    return -2;
  RecurArgs a{proj, ldp, q_off, k_off, v_off, gate, ldg, gate_off, gate2_off, bias, bias2, param, qscale, kscale, state, state_ld,
              out, ldo, seq_rows, slots, positions, heads, dim, vdim, chunks, scan_local, scan_start};
  hipStream_t s = (hipStream_t)stream;
  if (mode == RECUR_SCALAR_GATES) return launch_recurrence_passes<RECUR_SCALAR_GATES>(a, nseq, nchunks, spans, nspans, s);
  if (mode == RECUR_DECAY_PER_CHANNEL) return launch_recurrence_passes<RECUR_DECAY_PER_CHANNEL>(a, nseq, nchunks, spans, nspans, s);
  if (mode == RECUR_BONUS_DECAY) return launch_recurrence_passes<RECUR_BONUS_DECAY>(a, nseq, nchunks, spans, nspans, s);
  if (mode == RECUR_FIXED_DECAY) return launch_recurrence_passes<RECUR_FIXED_DECAY>(a, nseq, nchunks, spans, nspans, s);
  return -2;
}

extern "C" int bw_head_norm_gate(const float* o, int ldi, const float* weight, int wstride, const float* g, int ldg, int gate,
                                 void* out, int out_is_bf16, int ldo, const int32_t* positions, int rows, int heads, int vdim,
                                 float eps, void* stream) {
  if (rows <= 0) return 0;
  if (heads <= 0 || vdim <= 0 || ldi < heads * vdim || ldo < heads * vdim) return -2;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((rows * heads + 3) / 4), block(256);
  if (out_is_bf16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, block, 0, s, o, ldi, weight, wstride, g, ldg, gate, (bf16_t*)out,
                       ldo, positions, rows, heads, vdim, eps);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, block, 0, s, o, ldi, weight, wstride, g, ldg, gate, (float*)out,
                       ldo, positions, rows, heads, vdim, eps);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_glu(const float* gate_up, int ldg, void* h, int out_is_bf16, int rows, int inter, int act, float limit, float alpha,
                      const float* row_gate, int ld_row_gate, void* stream) {
  if (rows <= 0 || inter <= 0) return 0;
  if (act != ACT_SILU && act != ACT_GELU_TANH && act != ACT_CLAMPED_SWISH) return -2;
  if (ldg < 2 * inter || (act == ACT_CLAMPED_SWISH && !(limit > 0.0f))) return -2;
  const long long n = (long long)rows * inter;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (out_is_bf16) hipLaunchKernelGGL(glu_kernel<bf16_t>, grid, block, 0, s, gate_up, ldg, (bf16_t*)h, n, inter, act, limit, alpha, row_gate, ld_row_gate);
  else hipLaunchKernelGGL(glu_kernel<float>, grid, block, 0, s, gate_up, ldg, (float*)h, n, inter, act, limit, alpha, row_gate, ld_row_gate);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_rotate_halves_rows(float* x, int ldx, int rows, int heads, int dim, int rot, int sections, int off0, int off1,
                                     const float* cos_table, const float* sin_table, const int32_t* positions, void* stream) {
  if (rows <= 0 || rot == 0) return 0;
  if (heads <= 0 || dim <= 0 || rot < 0 || rot % 2 || rot > dim || sections < 1 || sections > 2) return -2;
  if (off0 < 0 || off0 + heads * dim > ldx || (sections == 2 && (off1 < 0 || off1 + heads * dim > ldx))) return -2;
  RotateRowsArgs a{x, ldx, rows, heads, dim, rot, sections, {off0, off1}, cos_table, sin_table, positions};
  const long long n = (long long)rows * sections * heads * (rot / 2);
  hipLaunchKernelGGL(rotate_halves_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, a);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_tanh_rows(float* x, int ld, int rows, int cols, void* stream) {
  if (rows <= 0 || cols <= 0) return 0;
  if (ld < cols) return -2;
  const long long n = (long long)rows * cols;
  hipLaunchKernelGGL(tanh_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, ld, rows, cols);
  return BW_LAUNCH_CHECK();
}
