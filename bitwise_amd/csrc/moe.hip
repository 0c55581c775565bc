// A feed-forward of routed experts.
//
//   route:    per row, scores = softmax of the router's logits over all experts, or the sigmoid of each; the choice is
//             made on the scores, or on the scores plus a learned correction per expert; experts lie in equal groups of
//             neighbours, a group's score is its best choice score (or the sum of its few best), only experts of the
//             `keep` best groups can be chosen; the `top` best of those are the row's experts, weighted by their scores
//             (without the correction) as they are.  Ties go to the lower index.  All 32-bit.
//   plan:     the step's (row, choice) pairs ("slots") sorted by expert into runs, and the runs cut into tiles of
//             16 or 128 slots (steps of few or of many slots): every tile belongs to one expert.  Built on the device; the products' grids are sized for
//             the worst case and tiles past the last return at once.
//   gate_up:  per tile, G = X W_gate^T and U = X W_up^T of its expert, then h = min(G, limit) * sigmoid(alpha * min(G, limit))
//             * (clamp(U, -limit, limit) + 1), stored by the slot's place in the sorted order
//   down:     per tile, h W_down^T of its expert, 32-bit sums by sorted place
//   combine:  out[row] = sum over the row's choices, in the order they were chosen, of weight * its expert's output
//
// bfloat16 mode runs the two products on the matrix cores (v_mfma_f32_16x16x32_bf16 over the inner size ascending from
// zero in steps of 64 elements, two instructions a step, one accumulator per 16 x 16 block of outputs): what a row gets depends on the row and its expert alone, not on
// the rows it shares a tile with.  The 32-bit mode runs one fused multiply-add chain per output over the inner size
// ascending.
#include <math.h>

#include "common.h"
#include "api.h"

#define MOE_TM 128           // slots a tile of a step with many slots
#define MOE_SMALL_SLOTS 1024  // steps of up to this many slots get tiles of 16
#define MOE_MAX_EXPERTS 1024

// ------------------------------------------------------------------------------ route

// (value, index) of the wave's best: larger value first, then lower index
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(v, off, 64);
    const int oi = __shfl_xor(i, off, 64);
    const bool take = ov > v || (ov == v && oi < i);
    v = take ? ov : v;
    i = take ? oi : i;
  }
}

// How a row's experts are scored and chosen.  kind 0: scores are the softmax of the logits over all experts; kind 1: the
// sigmoid of each logit.  correction (optional, [E]): the choice is made on score + correction, the weights stay the scores.
// group_best: a group's score is the sum of its group_best largest choice scores (1: its best expert's).
struct RouteRule {
  int kind;
  const float* correction;
  int group_best;
};

// A wave a row.  LDS of the wave: scores [E], choice scores [E], group scores [count], allowed [count].
__device__ __forceinline__ void route_row(const float* __restrict__ logits, int ld, int row, int E, int top, int count, int keep,
                                          float weight_scale, RouteRule rule, int32_t* __restrict__ ids, float* __restrict__ wts,
                                          float* s, int lane) {
  float* c = s + E;
  float* gs = c + E;
  float* allowed = gs + count;
  const float* z = logits + (size_t)row * ld;
  if (rule.kind == 1) {
    for (int e = lane; e < E; e += 64) s[e] = 1.0f / (1.0f + bw_expf(-z[e]));
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int e = lane; e < E; e += 64) {
      const float ex = bw_expf(z[e] - mx);
      s[e] = ex;
      sum += ex;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) s[e] = s[e] / sum;
  }
  for (int e = lane; e < E; e += 64) c[e] = rule.correction != nullptr ? s[e] + rule.correction[e] : s[e];
  __builtin_amdgcn_wave_barrier();
  const int gsz = E / count;
  for (int g = lane; g < count; g += 64) {
    // the group's largest choice scores, one after the other (lower index first among equals), added in that order
    float total = 0.0f;
    int taken[4] = {-1, -1, -1, -1};
    const int nbest = min(min(rule.group_best, gsz), 4);
    for (int b = 0; b < nbest; ++b) {
      float best = -INFINITY;
      int at = -1;
      for (int j = 0; j < gsz; ++j) {
        if (j == taken[0] || j == taken[1] || j == taken[2] || j == taken[3]) continue;
        if (at < 0 || c[g * gsz + j] > best) { best = c[g * gsz + j]; at = j; }
      }
      taken[b] = at;
      total = b == 0 ? best : total + best;
    }
    gs[g] = total;
    allowed[g] = keep >= count ? 1.0f : 0.0f;
  }
  __builtin_amdgcn_wave_barrier();
  if (keep < count) {
    for (int it = 0; it < keep; ++it) {
      float v = -INFINITY;
      int i = 0x7fffffff;
      for (int g = lane; g < count; g += 64)
        if (allowed[g] == 0.0f && (i == 0x7fffffff || gs[g] > v)) { v = gs[g]; i = g; }
      wave_argmax(v, i);
      if (lane == 0) allowed[i] = 1.0f;
      __builtin_amdgcn_wave_barrier();
    }
  }
  // (a chosen expert's choice score becomes NaN: no comparison takes it again)
  for (int it = 0; it < top; ++it) {
    float v = -INFINITY;
    int i = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const bool open = allowed[e / gsz] > 0.0f && c[e] == c[e];
      if (open && (i == 0x7fffffff || c[e] > v)) { v = c[e]; i = e; }
    }
    wave_argmax(v, i);
    if (lane == 0) {
      ids[(size_t)row * top + it] = i;
      wts[(size_t)row * top + it] = s[i] * weight_scale;
      c[i] = __builtin_nanf("");
    }
    __builtin_amdgcn_wave_barrier();
  }
}

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int ld, int rows, int E, int top, int count,
                                                        int keep, float weight_scale, RouteRule rule, int32_t* __restrict__ ids,
                                                        float* __restrict__ wts) {
  extern __shared__ float route_lds[];
  const int wave = wave_index(), lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + wave;
  if (row >= rows) return;
  route_row(logits, ld, row, E, top, count, keep, weight_scale, rule, ids, wts, route_lds + (size_t)wave * (2 * E + 2 * count), lane);
}

extern "C" int bw_moe_route(const float* logits, int ld, int rows, int experts, int top, int groups, int keep, float weight_scale,
                            int score_kind, const float* correction, int group_best, int32_t* ids, float* wts, void* stream) {
  if (rows <= 0) return 0;
  if (experts < 1 || experts > MOE_MAX_EXPERTS || top < 1 || groups < 1 || experts % groups || keep < 1 || keep > groups ||
      top > keep * (experts / groups) || score_kind < 0 || score_kind > 1 || group_best < 1 || group_best > 4)
    return -2;
  const size_t bytes = (size_t)4 * (2 * experts + 2 * groups) * sizeof(float);
  hipLaunchKernelGGL(moe_route_kernel, dim3((rows + 3) / 4), dim3(256), bytes, (hipStream_t)stream, logits, ld, rows, experts, top,
                     groups, keep, weight_scale, RouteRule{score_kind, correction, group_best}, ids, wts);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ plan

// One workgroup of 1024 threads.  sorted[p] = slot at sorted place p; place[slot] = p; tiles[t] = (expert, first place,
// slots, 0) with up to tm slots a tile; meta[0] = number of tiles.  Thread (segment g, expert e) walks segment g of the
// slots (from LDS, where the workgroup has put them if they fit) and counts those of expert e; after a prefix over
// segments and experts it walks the segment again and hands out places.  Within an expert's run the slots ascend, so
// the plan is the same from run to run.
__device__ __forceinline__ void plan_body(const int32_t* __restrict__ ids, int n, int E, int segs, int tm, int staged, int* plan_ids,
                                          int32_t* __restrict__ sorted, int32_t* __restrict__ place, int32_t* __restrict__ tiles,
                                          int32_t* __restrict__ meta) {
  __shared__ int seg_count[1024];       // [expert][segment]; after the prefix: slots of the expert in earlier segments
  __shared__ int counts[MOE_MAX_EXPERTS], start[MOE_MAX_EXPERTS], tile0[MOE_MAX_EXPERTS];
  const int tid = threadIdx.x;
  if (staged) {
    for (int sidx = tid; sidx < n; sidx += 1024) plan_ids[sidx] = ids[sidx];
    __syncthreads();
  }
  const int* src = staged ? plan_ids : ids;
  const int e = tid % E, g = tid / E;
  const int seg_len = (n + segs - 1) / segs;
  const int s0 = g * seg_len, s1 = min(n, s0 + seg_len);
  const bool mine = g < segs;
  if (mine) {
    int c = 0;
    for (int sidx = s0; sidx < s1; ++sidx) c += src[sidx] == e;
    seg_count[e * segs + g] = c;
  }
  __syncthreads();
  if (tid < E) {
    int c = 0;
    for (int k = 0; k < segs; ++k) {
      const int v = seg_count[tid * segs + k];
      seg_count[tid * segs + k] = c;
      c += v;
    }
    counts[tid] = c;
  }
  __syncthreads();
  if (tid == 0) {
    int p = 0, t = 0;
    for (int x = 0; x < E; ++x) {
      start[x] = p;
      tile0[x] = t;
      p += counts[x];
      t += (counts[x] + tm - 1) / tm;
    }
    meta[0] = t;
  }
  __syncthreads();
  if (mine) {
    int p = start[e] + seg_count[e * segs + g];
    for (int sidx = s0; sidx < s1; ++sidx)
      if (src[sidx] == e) {
        sorted[p] = sidx;
        place[sidx] = p;
        ++p;
      }
  }
  for (int x = tid; x < E; x += 1024) {
    const int nt = (counts[x] + tm - 1) / tm;
    for (int t = 0; t < nt; ++t) {
      int32_t* rec = tiles + (size_t)(tile0[x] + t) * 4;
      rec[0] = x;
      rec[1] = start[x] + t * tm;
      rec[2] = min(tm, counts[x] - t * tm);
      rec[3] = 0;
    }
  }
}

__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t* __restrict__ ids, int n, int E, int segs, int tm, int staged,
                                                        int32_t* __restrict__ sorted, int32_t* __restrict__ place,
                                                        int32_t* __restrict__ tiles, int32_t* __restrict__ meta) {
  extern __shared__ int plan_lds[];     // [n] if staged
  plan_body(ids, n, E, segs, tm, staged, plan_lds, sorted, place, tiles, meta);
}

// Steps of up to 16 rows: route (a wave a row) and plan in one launch of one workgroup.
__global__ __launch_bounds__(1024) void moe_route_plan_kernel(const float* __restrict__ logits, int ld, int rows, int E, int top, int count,
                                                              int keep, float weight_scale, RouteRule rule, int32_t* __restrict__ ids, float* __restrict__ wts, int segs,
                                                              int tm, int32_t* __restrict__ sorted, int32_t* __restrict__ place,
                                                              int32_t* __restrict__ tiles, int32_t* __restrict__ meta) {
  extern __shared__ float both_lds[];   // the waves' routing tables, then the plan's slots
  const int wave = wave_index(), lane = threadIdx.x & 63;
  if (wave < rows) route_row(logits, ld, wave, E, top, count, keep, weight_scale, rule, ids, wts, both_lds + (size_t)wave * (2 * E + 2 * count), lane);
  __syncthreads();                      // (the rows' choices, written to memory by their waves, are visible to the workgroup)
  plan_body(ids, rows * top, E, segs, tm, 1, reinterpret_cast<int*>(both_lds + (size_t)rows * (2 * E + 2 * count)), sorted, place, tiles, meta);
}

// Slots a tile: few slots a step (decoded tokens) get tiles of 16, whose kernel keeps many steps of weights in flight;
// prompt portions get tiles of 128, which a workgroup stages in LDS.
extern "C" int bw_moe_tile_rows(int slots) { return slots <= MOE_SMALL_SLOTS ? 16 : MOE_TM; }

extern "C" int bw_moe_max_tiles(int slots, int experts) {
  const int full = slots / bw_moe_tile_rows(slots);
  return full + (experts < slots ? experts : slots);
}

extern "C" int bw_moe_plan(const int32_t* ids, int slots, int experts, int32_t* sorted, int32_t* place, int32_t* tiles,
                           int32_t* meta, void* stream) {
  if (slots <= 0) return 0;
  if (experts < 1 || experts > MOE_MAX_EXPERTS) return -2;
  const int segs = 1024 / experts;
  const int staged = slots <= 12 * 1024;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), staged ? (size_t)slots * sizeof(int) : 0, (hipStream_t)stream, ids, slots,
                     experts, segs, bw_moe_tile_rows(slots), staged, sorted, place, tiles, meta);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_moe_route_plan(const float* logits, int ld, int rows, int experts, int top, int groups, int keep,
                                 float weight_scale, int score_kind, const float* correction, int group_best, int32_t* ids, float* wts,
                                 int32_t* sorted, int32_t* place, int32_t* tiles, int32_t* meta, void* stream) {
  if (rows <= 0) return 0;
  const size_t bytes = ((size_t)rows * (2 * experts + 2 * groups) + (size_t)rows * top) * sizeof(float);
  if (rows > 16 || bytes > 48 * 1024) {
    const int rc = bw_moe_route(logits, ld, rows, experts, top, groups, keep, weight_scale, score_kind, correction, group_best, ids, wts, stream);
    return rc != 0 ? rc : bw_moe_plan(ids, rows * top, experts, sorted, place, tiles, meta, stream);
  }
  if (experts < 1 || experts > MOE_MAX_EXPERTS || top < 1 || groups < 1 || experts % groups || keep < 1 || keep > groups ||
      top > keep * (experts / groups) || score_kind < 0 || score_kind > 1 || group_best < 1 || group_best > 4)
    return -2;
  hipLaunchKernelGGL(moe_route_plan_kernel, dim3(1), dim3(1024), bytes, (hipStream_t)stream, logits, ld, rows, experts, top, groups, keep,
                     weight_scale, RouteRule{score_kind, correction, group_best}, ids, wts, 1024 / experts, bw_moe_tile_rows(rows * top), sorted, place, tiles, meta);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ the experts' activation

__device__ __forceinline__ float moe_act(float g, float u, float limit, float alpha) {
  if (!(limit > 0.0f)) return (g * (1.0f / (1.0f + bw_expf(-alpha * g)))) * u;      // the plain gated form
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return (g * (1.0f / (1.0f + bw_expf(-alpha * g)))) * (u + 1.0f);
}

// ------------------------------------------------------------------------------ products on the matrix cores

struct MoeArgs {
  const int32_t* sorted;   // [slots]
  const int32_t* tiles;    // [max_tiles][4]
  const int32_t* meta;
  int top, K, N;           // inner size, output columns of the product (ff for gate_up, width for down)
  float limit, alpha;
};

// A workgroup of four waves per (tile of 16 MB slots, 128 output columns); a wave owns 32 columns, for GATE_UP of
// the gate and of the up matrix both, and all of the tile's rows.  Operands go from memory straight into registers: lane
// (r, g) holds row r's (or column r's) elements k + 8g .. k + 8g + 7; a ring of DEPTH sets of operand registers keeps as
// many steps of the inner size in flight.  MB blocks of 16 rows a tile: 1 with a deep ring for the few rows of decoded
// tokens, where the weights stream from memory once and nothing is reused (prompt portions: moe_lds_kernel below).  Blocks of 16 rows past the tile's slots are skipped (a scalar
// branch: the matrix cores ignore the execution mask); rows past them inside a block read the tile's first row and are
// never stored.
template <bool GATE_UP, int MB, int DEPTH, int CW>
__global__ __launch_bounds__(256) void moe_mfma_kernel(MoeArgs a, const bf16_t* __restrict__ x, int ldx, int x_rows,
                                                       const bf16_t* __restrict__ w, void* __restrict__ out, int ldo, int max_tiles) {
  // Workgroups are dealt to the chip's eight dies in turn, and every die has an L2 of its own.  Workgroup L is the
  // (L / 8)-th of die L % 8; a die takes the blocks of 128 columns c = die, die + 8, ... and, for each, walks the tiles
  // in order: tiles of one expert follow each other, so a block of an expert's weights is fetched into one L2 once and
  // serves all of the expert's tiles from there.
  const int die = blockIdx.x & 7, nth = blockIdx.x >> 3;
  const int tile = nth % max_tiles, col_block = die + 8 * (nth / max_tiles);
  if (tile >= a.meta[0] || col_block * (4 * CW) >= a.N) return;
  const int wave = wave_index(), lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int e = __builtin_amdgcn_readfirstlane(a.tiles[tile * 4]), p0 = __builtin_amdgcn_readfirstlane(a.tiles[tile * 4 + 1]),
            cnt = __builtin_amdgcn_readfirstlane(a.tiles[tile * 4 + 2]);
  const int n0 = col_block * (4 * CW) + wave * CW;         // CW columns a wave (32, or 16 where a step has very few slots
  if (n0 >= a.N) return;                                   // and more workgroups are worth more than wider ones)
  constexpr int CB = CW / 16, NB = GATE_UP ? 2 * CB : CB;
  const int mb_live = (cnt + 15) >> 4;                     // blocks of 16 rows that hold a slot
  // Every load goes through a buffer descriptor with a per-lane offset fixed for the whole kernel and the step's offset
  // in a scalar register: the loop spends no vector instruction on addresses and no branch on a load.  Rows of x are
  // gathered (a lane's offset names its slot's row); lanes of row blocks without slots and of weight rows past the
  // matrix point outside their descriptors, read zeros and ask memory for nothing.
  const int K = a.K;
  const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)((size_t)x_rows * ldx * 2), 0x00020000);
  int voff_x[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int q = 16 * i + r;
    const int pq = p0 + (q < cnt ? q : 0);
    const size_t row = GATE_UP ? (size_t)(a.sorted[pq] / a.top) : (size_t)pq;
    voff_x[i] = i < mb_live ? (int)((row * ldx + 16 * g) * 2) : 0x7ffffff0;
  }
  // weights of expert e: GATE_UP [2N, K] (gate rows, then up rows), else [N, K]
  __amdgpu_buffer_rsrc_t rs_w[NB];
  const size_t wbase = (size_t)e * (GATE_UP ? 2 : 1) * a.N * a.K;
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int half = GATE_UP ? b / CB : 0, cb = GATE_UP ? b % CB : b;
    const int nb0 = n0 + 16 * cb;
    const int rows_in = min(16, a.N - nb0);                // (may be <= 0: then nothing of the block is read)
    rs_w[b] = __builtin_amdgcn_make_buffer_rsrc((void*)(w + wbase + ((size_t)half * a.N + (rows_in > 0 ? nb0 : 0)) * a.K), 0,
                                                rows_in > 0 ? (int)((size_t)rows_in * a.K * 2) : 0, 0x00020000);
  }
  const int voff_w = (r * K + 16 * g) * 2;
  f32x4 acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[i][b] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const bool tail = (K & 63) != 0;                         // (scalar)
  // A step covers 64 elements of the inner size: lane (r, g) holds elements k + 16g .. k + 16g + 15 of its row, 32
  // contiguous bytes, so that a wave's loads take whole 128-byte lines; the first matrix instruction of the step
  // multiplies every lane's first eight elements, the second its last eight (which elements meet in which instruction
  // is the same for both operands and for every tile shape, so the sums' bits do not depend on the shape).
  struct Ops { u32x4 af[MB][2], bfr[NB][2]; };
  auto load = [&](int k, Ops& o) {
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      o.af[i][0] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff_x[i], k * 2, 0);
      o.af[i][1] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff_x[i], k * 2 + 16, 0);
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      o.bfr[b][0] = __builtin_amdgcn_raw_buffer_load_b128(rs_w[b], voff_w, k * 2, 0);
      o.bfr[b][1] = __builtin_amdgcn_raw_buffer_load_b128(rs_w[b], voff_w, k * 2 + 16, 0);
    }
  };
  auto mma = [&](int k, const Ops& o) {
#pragma unroll
    for (int hlf = 0; hlf < 2; ++hlf) {
      // (an inner size that is no multiple of 64: what a lane holds past K came from the next row, and counts as zero)
      const bool live = !tail || k + 16 * g + 8 * hlf + 8 <= K;
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        if (i < mb_live) {                                 // scalar
          const u32x4 av = live ? o.af[i][hlf] : zero;
#pragma unroll
          for (int b = 0; b < NB; ++b)
            acc[i][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(av), as_bf16x8(live ? o.bfr[b][hlf] : zero), acc[i][b], 0, 0, 0);
        }
      }
    }
  };
  Ops ring[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load(64 * d, ring[d]);
  __builtin_amdgcn_sched_barrier(0);
  for (int k = 0; k < K; k += 64 * DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (k + 64 * d < K) {                                // (scalar)
        mma(k + 64 * d, ring[d]);
        // the refill stays where it is written: left to itself the scheduler moves every load to just before its
        // use, and the ring holds nothing in flight
        __builtin_amdgcn_sched_barrier(0);
        load(k + 64 * (d + DEPTH), ring[d]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // accumulator element q of block (i, b): slot 16 i + 4 g + q, column 16 b' + r
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = 16 * i + 4 * g + q;
      if (m >= cnt) continue;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const int n = n0 + 16 * cb + r;
        if (n >= a.N) continue;
        if constexpr (GATE_UP)
          reinterpret_cast<bf16_t*>(out)[(size_t)(p0 + m) * ldo + n] = f32_to_bf16(moe_act(acc[i][cb][q], acc[i][CB + cb][q], a.limit, a.alpha));
        else
          reinterpret_cast<float*>(out)[(size_t)(p0 + m) * ldo + n] = acc[i][cb][q];
      }
    }
}

// ------------------------------------------------------------------------------ prompt portions: tiles staged in LDS

// A workgroup of four waves per (tile of 128 slots, 128 output columns; GATE_UP: of the gate and of the up matrix both,
// 256 weight rows).  A step covers 64 elements of the inner size: the threads together copy the tile's 128 rows of x and
// its weight rows, 128 bytes each, from memory into LDS (through registers: the next step's loads fly while this one is
// multiplied; two stages, one barrier a step; rows 144 bytes apart against bank conflicts), and wave (wr, wc) multiplies
// rows 64 wr .. of the tile by columns 64 wc .. of the block from there.  A lane reads from LDS exactly the elements it
// would have loaded itself in moe_mfma_kernel, so the same elements meet in the same matrix instruction and the sums
// have the same bits as there.  87 flops for every byte that comes from L2, against 32 when every wave loads for itself.
#define MOE_LDS_STRIDE 144

template <bool GATE_UP>
__global__ __launch_bounds__(256) void moe_lds_kernel(MoeArgs a, const bf16_t* __restrict__ x, int ldx, int x_rows,
                                                      const bf16_t* __restrict__ w, void* __restrict__ out, int ldo, int max_tiles) {
  constexpr int TM = MOE_TM, BR = GATE_UP ? 256 : 128, ROWS = TM + BR;
  constexpr int NCH = ROWS * 8 / 256;                       // 16-byte chunks a thread copies a step
  constexpr int STAGE = ROWS * MOE_LDS_STRIDE;
  constexpr int NB = GATE_UP ? 8 : 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char moe_lds[];
  const int die = blockIdx.x & 7, nth = blockIdx.x >> 3;
  const int tile = nth % max_tiles, col_block = die + 8 * (nth / max_tiles);
  if (tile >= a.meta[0] || col_block * 128 >= a.N) return;
  const int wave = wave_index(), lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4, tid = threadIdx.x;
  const int wr = wave >> 1, wc = wave & 1;
  const int e = __builtin_amdgcn_readfirstlane(a.tiles[tile * 4]), p0 = __builtin_amdgcn_readfirstlane(a.tiles[tile * 4 + 1]),
            cnt = __builtin_amdgcn_readfirstlane(a.tiles[tile * 4 + 2]);
  const int n0 = col_block * 128;
  const int K = a.K;
  const bool tail = (K & 63) != 0;
  const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)((size_t)x_rows * ldx * 2), 0x00020000);
  const size_t wbase = (size_t)e * (GATE_UP ? 2 : 1) * a.N * a.K;
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc((void*)(w + wbase), 0, (int)((size_t)(GATE_UP ? 2 : 1) * a.N * a.K * 2), 0x00020000);
  // chunk c = tid + 256 j: row c / 8 of the stage (x rows first, then weight rows), bytes 16 (c % 8) .. of the row's step
  int voff[NCH], lds_off[NCH];
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int c = tid + 256 * j, row = c >> 3, part = c & 7;
    lds_off[j] = row * MOE_LDS_STRIDE + part * 16;
    if (row < TM) {
      const int pq = p0 + (row < cnt ? row : 0);
      const size_t src = GATE_UP ? (size_t)(a.sorted[pq] / a.top) : (size_t)pq;
      voff[j] = (int)((src * ldx) * 2) + part * 16;
    } else {
      const int br = row - TM, half = GATE_UP ? br >> 7 : 0;
      const int n = min(n0 + (br & 127), a.N - 1);
      voff[j] = (int)(((size_t)half * a.N + n) * a.K * 2) + part * 16;
    }
  }
  const u32x4 zero = {0u, 0u, 0u, 0u};
  // two sets of registers: the loads of the next step and of the one after it are in flight while a step is multiplied
  // (every weight comes from memory once, so what hides the memory's latency is the bytes a compute unit has asked for)
  u32x4 regs_a[NCH], regs_b[NCH];
  auto fetch = [&](int k, u32x4 (&regs)[NCH]) {
    if (k >= K) return;                                    // (scalar)
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      // (a thread's chunk j lies in rows 32 j .. 32 j + 31: x rows for the first TM / 32 chunks, weight rows after)
      regs[j] = j < TM / 32 ? __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff[j], k * 2, 0)
                            : __builtin_amdgcn_raw_buffer_load_b128(rs_w, voff[j], k * 2, 0);
    }
  };
  auto stash = [&](int k, int stage, const u32x4 (&regs)[NCH]) {
    if (k >= K) return;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int part = (tid + 256 * j) & 7;
      const u32x4 v = (!tail || k + 8 * part < K) ? regs[j] : zero;       // (past K a chunk counts as zero)
      *reinterpret_cast<u32x4*>(moe_lds + stage * STAGE + lds_off[j]) = v;
    }
  };
  f32x4 acc[4][NB];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[i][b] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const int mb_live = min(4, max(0, (cnt - 64 * wr + 15) >> 4));      // this wave's blocks of 16 rows that hold a slot
  const int a_off = (64 * wr + r) * MOE_LDS_STRIDE + 32 * g;
  int b_off[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int half = GATE_UP ? b >> 2 : 0, cb = b & 3;
    b_off[b] = (TM + 128 * half + 64 * wc + 16 * cb + r) * MOE_LDS_STRIDE + 32 * g;
  }
  auto multiply = [&](int stage) {
    const unsigned char* base = moe_lds + stage * STAGE;
#pragma unroll
    for (int hlf = 0; hlf < 2; ++hlf) {
      u32x4 bf[NB];
#pragma unroll
      for (int b = 0; b < NB; ++b) bf[b] = *reinterpret_cast<const u32x4*>(base + b_off[b] + 16 * hlf);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (i < mb_live) {                                 // scalar
          const u32x4 af = *reinterpret_cast<const u32x4*>(base + a_off + 16 * i * MOE_LDS_STRIDE + 16 * hlf);
#pragma unroll
          for (int b = 0; b < NB; ++b)
            acc[i][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(af), as_bf16x8(bf[b]), acc[i][b], 0, 0, 0);
        }
      }
    }
  };
  fetch(0, regs_a);
  fetch(64, regs_b);
  stash(0, 0, regs_a);
  fetch(128, regs_a);
  __syncthreads();
  // step k is multiplied from stage 0 while regs_b (step k + 64) goes to stage 1 and is asked for again three steps ahead;
  // then the same with the roles swapped
  for (int k = 0; k < K; k += 128) {
    multiply(0);
    stash(k + 64, 1, regs_b);
    fetch(k + 192, regs_b);
    __syncthreads();
    if (k + 64 < K) {                                      // (scalar)
      multiply(1);
      stash(k + 128, 0, regs_a);
      fetch(k + 256, regs_a);
      __syncthreads();
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = 64 * wr + 16 * i + 4 * g + q;
      if (m >= cnt) continue;
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) {
        const int n = n0 + 64 * wc + 16 * cb + r;
        if (n >= a.N) continue;
        if constexpr (GATE_UP)
          reinterpret_cast<bf16_t*>(out)[(size_t)(p0 + m) * ldo + n] = f32_to_bf16(moe_act(acc[i][cb][q], acc[i][4 + cb][q], a.limit, a.alpha));
        else
          reinterpret_cast<float*>(out)[(size_t)(p0 + m) * ldo + n] = acc[i][cb][q];
      }
    }
}

template <bool GATE_UP>
static int moe_lds_launch(const MoeArgs& a, const bf16_t* x, int ldx, int x_rows, const bf16_t* w, void* out, int ldo, int max_tiles,
                          hipStream_t s) {
  constexpr int BYTES = 2 * (MOE_TM + (GATE_UP ? 256 : 128)) * MOE_LDS_STRIDE;
  static bool allowed = false;
  if (!allowed) {
    if (hipFuncSetAttribute((const void*)moe_lds_kernel<GATE_UP>, hipFuncAttributeMaxDynamicSharedMemorySize, BYTES) != hipSuccess) return -8;
    allowed = true;
  }
  const int col_blocks = (a.N + 127) / 128;
  hipLaunchKernelGGL(moe_lds_kernel<GATE_UP>, dim3((unsigned)(8 * ((col_blocks + 7) / 8) * max_tiles)), dim3(256), BYTES, s, a, x, ldx, x_rows,
                     w, out, ldo, max_tiles);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ products in 32-bit

// A thread an output (sorted place, column): one chain of fused multiply-adds over the inner size ascending.
// ROUND: the activation is rounded to bfloat16 (and kept as a 32-bit value), for the bfloat16 mode of weights that the
// matrix-core kernels do not take.
template <bool GATE_UP, typename WT>
__global__ __launch_bounds__(64) void moe_f32_kernel(MoeArgs a, const float* __restrict__ x, int ldx, const WT* __restrict__ w,
                                                     float* __restrict__ out, int ldo, int round_out) {
  const int tile = blockIdx.x;
  if (tile >= a.meta[0]) return;
  const int e = a.tiles[tile * 4], p0 = a.tiles[tile * 4 + 1], cnt = a.tiles[tile * 4 + 2];
  const int n = blockIdx.y * 64 + threadIdx.x;
  if (n >= a.N) return;
  const size_t wbase = (size_t)e * (GATE_UP ? 2 : 1) * a.N * a.K;
  const WT* wg = w + wbase + (size_t)n * a.K;
  const WT* wu = wg + (size_t)a.N * a.K;
  for (int m = 0; m < cnt; ++m) {
    const float* xr = x + (GATE_UP ? (size_t)(a.sorted[p0 + m] / a.top) : (size_t)(p0 + m)) * ldx;
    float sg = 0.0f, su = 0.0f;
    for (int k = 0; k < a.K; ++k) {
      const float xv = xr[k];
      if constexpr (sizeof(WT) == 2) {
        sg = fmaf(xv, bf16_to_f32(wg[k]), sg);
        if (GATE_UP) su = fmaf(xv, bf16_to_f32(wu[k]), su);
      } else {
        sg = fmaf(xv, wg[k], sg);
        if (GATE_UP) su = fmaf(xv, wu[k], su);
      }
    }
    float y = GATE_UP ? moe_act(sg, su, a.limit, a.alpha) : sg;
    if (GATE_UP && round_out) y = bf16_to_f32(f32_to_bf16(y));
    out[(size_t)(p0 + m) * ldo + n] = y;
  }
}

extern "C" int bw_moe_experts(const void* x, int x_is_bf16, int ldx, int x_rows, const void* w, int w_is_bf16, void* out, int ldo,
                              const int32_t* sorted, const int32_t* tiles, const int32_t* meta, int slots, int max_tiles, int top,
                              int K, int N, int gate_up, float limit, float alpha, int round_out, void* stream) {
  const int tile_rows = bw_moe_tile_rows(slots);          // (as the plan was made)
  if (max_tiles <= 0 || slots <= 0) return 0;
  if (K <= 0 || N <= 0 || (N + 63) / 64 > 65535) return -2;
  MoeArgs a{sorted, tiles, meta, top, K, N, limit, alpha};
  hipStream_t s = (hipStream_t)stream;
  if (x_is_bf16) {
    if (!w_is_bf16 || K % 8 || ldx % 8) return -3;
    if ((size_t)x_rows * ldx * 2 >= (1ull << 31) || (size_t)16 * K * 2 >= (1ull << 31)) return -2;      // offsets inside a descriptor are 32-bit
    if (tile_rows == 16) {
      // very few slots (a step of up to 16 rows of four experts): 16 columns a wave, twice the workgroups
      const int cw = slots <= 64 ? 16 : 32;
      const int col_blocks = (N + 4 * cw - 1) / (4 * cw);
      const dim3 grid((unsigned)(8 * ((col_blocks + 7) / 8) * max_tiles));
      if (cw == 16) {
        if (gate_up) hipLaunchKernelGGL((moe_mfma_kernel<true, 1, 6, 16>), grid, dim3(256), 0, s, a, (const bf16_t*)x, ldx, x_rows, (const bf16_t*)w, out, ldo, max_tiles);
        else hipLaunchKernelGGL((moe_mfma_kernel<false, 1, 8, 16>), grid, dim3(256), 0, s, a, (const bf16_t*)x, ldx, x_rows, (const bf16_t*)w, out, ldo, max_tiles);
      } else {
        if (gate_up) hipLaunchKernelGGL((moe_mfma_kernel<true, 1, 4, 32>), grid, dim3(256), 0, s, a, (const bf16_t*)x, ldx, x_rows, (const bf16_t*)w, out, ldo, max_tiles);
        else hipLaunchKernelGGL((moe_mfma_kernel<false, 1, 6, 32>), grid, dim3(256), 0, s, a, (const bf16_t*)x, ldx, x_rows, (const bf16_t*)w, out, ldo, max_tiles);
      }
    } else {
      if ((size_t)2 * N * K * 2 >= (1ull << 31)) return -2;
      return gate_up ? moe_lds_launch<true>(a, (const bf16_t*)x, ldx, x_rows, (const bf16_t*)w, out, ldo, max_tiles, s)
                     : moe_lds_launch<false>(a, (const bf16_t*)x, ldx, x_rows, (const bf16_t*)w, out, ldo, max_tiles, s);
    }
    return BW_LAUNCH_CHECK();
  }
  const dim3 grid(max_tiles, (N + 63) / 64);
  if (gate_up) {
    if (w_is_bf16) hipLaunchKernelGGL((moe_f32_kernel<true, bf16_t>), grid, dim3(64), 0, s, a, (const float*)x, ldx, (const bf16_t*)w, (float*)out, ldo, round_out);
    else hipLaunchKernelGGL((moe_f32_kernel<true, float>), grid, dim3(64), 0, s, a, (const float*)x, ldx, (const float*)w, (float*)out, ldo, round_out);
  } else {
    if (w_is_bf16) hipLaunchKernelGGL((moe_f32_kernel<false, bf16_t>), grid, dim3(64), 0, s, a, (const float*)x, ldx, (const bf16_t*)w, (float*)out, ldo, 0);
    else hipLaunchKernelGGL((moe_f32_kernel<false, float>), grid, dim3(64), 0, s, a, (const float*)x, ldx, (const float*)w, (float*)out, ldo, 0);
  }
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------ combine

// out[row][c] (=, or +=) sum_j wts[row][j] * y[place[row * top + j]][c], j ascending, one chain per element.
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, int ldy, const int32_t* __restrict__ place,
                                                          const float* __restrict__ wts, int top, float* __restrict__ out, int ldo,
                                                          int width, int accumulate) {
  const int row = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= width) return;
  float acc = 0.0f;
  for (int j = 0; j < top; ++j)
    acc = fmaf(wts[(size_t)row * top + j], y[(size_t)place[(size_t)row * top + j] * ldy + c], acc);
  float* o = out + (size_t)row * ldo + c;
  *o = accumulate ? *o + acc : acc;
}

extern "C" int bw_moe_combine(const float* y, int ldy, const int32_t* place, const float* wts, int top, float* out, int ldo,
                              int rows, int width, int accumulate, void* stream) {
  if (rows <= 0) return 0;
  if (rows > 65535) return -2;
  hipLaunchKernelGGL(moe_combine_kernel, dim3((width + 255) / 256, rows), dim3(256), 0, (hipStream_t)stream, y, ldy, place, wts, top,
                     out, ldo, width, accumulate);
  return BW_LAUNCH_CHECK();
}
