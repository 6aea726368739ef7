// Products whose weight depends on the row's group: a matrix per head (out[t, h, :] = W_h a[t, h, :]) and a
// matrix per expert for the rows that a router sent there; the router's choice and the plan that sorts a step's
// (row, choice) pairs by expert.  bfloat16 products run on the matrix cores (v_mfma_f32_16x16x32_bf16, operands
// straight from memory into the lanes that the instruction reads; the experts' matrices packed in that order);
// 32-bit products, and sizes the matrix-core kernels do not take, run in one tiled vector routine (16 rows x 64
// columns a workgroup, K in chunks of 32 through LDS).  Every kernel sums an output's k in one ascending order,
// so a row's result does not depend on which other rows share its tile or on which kernel variant ran.
#include "common.h"

namespace {

__device__ __forceinline__ float load_as(const void* p, size_t i, int dt) {
  return dt == DN_F32 ? static_cast<const float*>(p)[i] : to_float(static_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void store_as(void* p, size_t i, int dt, float v) {
  if (dt == DN_F32) static_cast<float*>(p)[i] = v;
  else static_cast<bf16_t*>(p)[i] = from_float<bf16_t>(v);
}

constexpr int TM = 16, TN = 64, TK = 32;

struct Tile {
  float a[TM][TK + 1];
  float w[TN][TK + 1];
};

// acc[c] (c < 4) += sum_k A[row, k] * W[n0 + cq * 4 + c, k] for this thread's row `tid / 16` and columns cq = tid % 16.
// a_row[q]: element offset of row tid / 32 + 8 q of the tile in A, or -1 where the tile has no such row.
// DUAL: a second weight W2 with its own sums.
template <bool DUAL>
__device__ __forceinline__ void tile_product(Tile& lds, Tile* lds2, const void* A, int a_dt, const long long a_row[2], const void* W,
                                             const void* W2, int w_dt, size_t w_base, int N, int K, int n0, float acc[4],
                                             float acc2[4]) {
  const int tid = threadIdx.x;
  const int lr = tid >> 5, lk = tid & 31;      // loads: row (or column of W) and k
  const int r = tid >> 4, cq = tid & 15;       // sums
  for (int k0 = 0; k0 < K; k0 += TK) {
    const bool kin = k0 + lk < K;
#pragma unroll
    for (int q = 0; q < 2; ++q)
      lds.a[lr + 8 * q][lk] = (kin && a_row[q] >= 0) ? load_as(A, static_cast<size_t>(a_row[q]) + k0 + lk, a_dt) : 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int n = n0 + lr + 8 * q;
      const bool ok = kin && n < N;
      const size_t at = w_base + static_cast<size_t>(n) * K + k0 + lk;
      lds.w[lr + 8 * q][lk] = ok ? load_as(W, at, w_dt) : 0.f;
      if (DUAL) lds2->w[lr + 8 * q][lk] = ok ? load_as(W2, at, w_dt) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      const float av = lds.a[r][kk];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        acc[c] = fmaf(av, lds.w[cq * 4 + c][kk], acc[c]);
        if (DUAL) acc2[c] = fmaf(av, lds2->w[cq * 4 + c][kk], acc2[c]);
      }
    }
    __syncthreads();
  }
}

// ---- a matrix per head ---------------------------------------------------------------------------------------
// out[t, o_off + h * o_stride + n] = sum_k W[h][n][k] * a[t, a_off + h * a_stride + k]
__global__ __launch_bounds__(256) void heads_linear_kernel(const void* A, int a_dt, size_t lda, int a_off, int a_stride, const void* W,
                                                           int w_dt, void* out, int out_dt, size_t ldo, int o_off, int o_stride,
                                                           int T, int N, int K) {
  __shared__ Tile lds;
  const int h = blockIdx.z, t0 = blockIdx.x * TM, n0 = blockIdx.y * TN;
  const int tid = threadIdx.x;
  long long a_row[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int t = t0 + (tid >> 5) + 8 * q;
    a_row[q] = t < T ? static_cast<long long>(t) * lda + a_off + static_cast<long long>(h) * a_stride : -1;
  }
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  tile_product<false>(lds, nullptr, A, a_dt, a_row, W, nullptr, w_dt, static_cast<size_t>(h) * N * K, N, K, n0, acc, nullptr);
  const int t = t0 + (tid >> 4);
  if (t >= T) return;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int n = n0 + (tid & 15) * 4 + c;
    if (n < N) store_as(out, static_cast<size_t>(t) * ldo + o_off + static_cast<size_t>(h) * o_stride + n, out_dt, acc[c]);
  }
}

// ---- the router's choice -------------------------------------------------------------------------------------
// Per row: s = softmax(z) over the experts; the `top` largest of s + correction are chosen (the lower index wins a
// tie), weighed by their s divided by the sum of the chosen s (+ 1e-20).  A thread a row.
// (sigmoid: the scores are s = 1 / (1 + e^-z), each expert's own; renorm 0: the weights are the chosen scores as they are.
// A row of z may be wider than the experts: rows are ldz numbers apart.)
__device__ __forceinline__ float route_score(bool sigmoid, float z, float m, float sum) {
  return sigmoid ? 1.0f / (1.0f + expf(-z)) : expf(z - m) / sum;
}

__global__ __launch_bounds__(64) void route_kernel(const float* z, size_t ldz, const float* correction, int T, int E, int top,
                                                   int sigmoid, int renorm, int* ids, float* wts) {
  const int t = blockIdx.x * 64 + threadIdx.x;
  if (t >= T) return;
  const float* row = z + static_cast<size_t>(t) * ldz;
  float m = row[0];
  for (int e = 1; e < E; ++e) m = fmaxf(m, row[e]);
  float sum = 0.f;
  for (int e = 0; e < E; ++e) sum += expf(row[e] - m);
  float chosen_sum = 0.f;
  for (int c = 0; c < top; ++c) {
    int best = -1;
    float best_v = 0.f, best_s = 0.f;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int q = 0; q < c; ++q) taken |= ids[t * top + q] == e;
      if (taken) continue;
      const float sc = route_score(sigmoid, row[e], m, sum);
      const float v = sc + (correction ? correction[e] : 0.f);
      if (best < 0 || v > best_v) best = e, best_v = v, best_s = sc;
    }
    ids[t * top + c] = best;
    wts[t * top + c] = best_s;
    chosen_sum += best_s;
  }
  if (!renorm) return;
  const float inv = 1.0f / (chosen_sum + 1e-20f);
  for (int c = 0; c < top; ++c) wts[t * top + c] *= inv;
}

// The same choice with a wave a row (up to 8,192 experts, `top` up to 64): lane l has the experts l, l + 64, ...; the
// largest score is found over the lanes, the lowest index among equals wins, and lane c keeps the c-th choice.
// groups > 1: the experts are `groups` equal runs of neighbours; a group's score is the sum of its two largest
// s + correction (of its one, if it has one expert), and only the experts of the `keep` best groups (the lower index wins a
// tie) can be chosen.  scale multiplies the weights.
__global__ __launch_bounds__(64) void route_wave_kernel(const float* z, size_t ldz, const float* correction, int E, int top, int sigmoid,
                                                        int renorm, int* ids, float* wts, int groups, int keep, float scale) {
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* row = z + static_cast<size_t>(t) * ldz;
  const float none = -__builtin_huge_valf();
  __shared__ unsigned char open_group[8192];      // (groups <= experts <= 8,192)
  __shared__ float group_score[8192];
  float m = none;
  for (int e = lane; e < E; e += 64) m = fmaxf(m, row[e]);
  m = wave_max(m);
  float sum = 0.f;
  for (int e = lane; e < E; e += 64) sum += expf(row[e] - m);
  sum = wave_sum(sum);
  unsigned taken[4] = {0u, 0u, 0u, 0u};      // a bit for each of the lane's up to 128 experts
  const int per = groups > 1 ? E / groups : E;
  if (groups > 1) {
    // lane l scores the groups l, l + 64, ...; then the best group is found `keep` times over the lanes
    for (int g = lane; g < groups; g += 64) {
      float first = none, second = none;
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float v = route_score(sigmoid, row[e], m, sum) + (correction ? correction[e] : 0.f);
        if (v > first) second = first, first = v;
        else if (v > second) second = v;
      }
      group_score[g] = per > 1 ? first + second : first;
      open_group[g] = 0;
    }
    __syncthreads();
    for (int c = 0; c < keep; ++c) {
      float best_v = none;
      int best = 0x7fffffff;
      for (int g = lane; g < groups; g += 64)
        if (!open_group[g] && group_score[g] > best_v) best_v = group_score[g], best = g;
      const float top_v = wave_max(best_v);
      int win = static_cast<int>(-wave_max(-static_cast<float>((best_v == top_v && best < groups) ? best : 16777216)));
      if (win >= groups) {      // (scores that are no numbers: the first group that is still closed)
        win = 0;
        while (win < groups - 1 && open_group[win]) ++win;
      }
      __syncthreads();
      if (lane == 0) open_group[win] = 1;
      __syncthreads();
    }
  }
  float my_w = 0.f;
  int my_id = 0;
  for (int c = 0; c < top; ++c) {
    float best_v = none, best_s = 0.f;
    int best = 0x7fffffff;
    for (int e = lane, k = 0; e < E; e += 64, ++k) {
      if ((taken[k >> 5] >> (k & 31)) & 1u) continue;
      if (groups > 1 && !open_group[e / per]) continue;
      const float sc = route_score(sigmoid, row[e], m, sum);
      const float v = sc + (correction ? correction[e] : 0.f);
      if (v > best_v) best_v = v, best = e, best_s = sc;
    }
    const float top_v = wave_max(best_v);
    int win = static_cast<int>(-wave_max(-static_cast<float>((best_v == top_v && best < E) ? best : 16777216)));
    if (win >= E) win = c;      // (scores that are no numbers: any expert, never an index outside)
    const bool mine = (win & 63) == lane;
    const float s_win = wave_max((mine && best == win) ? best_s : none);
    if (mine) taken[(win >> 6) >> 5] |= 1u << ((win >> 6) & 31);
    if (lane == c) my_id = win, my_w = s_win > none ? s_win : 0.f;
  }
  const float chosen = wave_sum(lane < top ? my_w : 0.f);
  if (lane < top) {
    ids[t * top + lane] = my_id;
    wts[t * top + lane] = (renorm ? my_w / (chosen + 1e-20f) : my_w) * scale;
  }
}

// ---- the plan ------------------------------------------------------------------------------------------------
// The n pairs (row, choice), pair i = row * top + choice, sorted by expert and inside an expert by i:
// offsets[e] .. offsets[e + 1] - 1 are expert e's places in `order`.  One workgroup.
__global__ __launch_bounds__(256) void plan_kernel(const int* ids, int n, int E, int* offsets, int* order) {
  extern __shared__ int shm[];
  int* base = shm;         // [E]
  int* cid = shm + E;      // [256]
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 256) base[e] = 0;
  __syncthreads();
  for (int i = tid; i < n; i += 256) atomicAdd(&base[ids[i]], 1);
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      const int c = base[e];
      offsets[e] = run;
      base[e] = run;
      run += c;
    }
    offsets[E] = run;
  }
  __syncthreads();
  for (int c0 = 0; c0 < n; c0 += 256) {
    const int i = c0 + tid;
    const int e = i < n ? ids[i] : -1;
    cid[tid] = e;
    __syncthreads();
    if (e >= 0) {
      int rank = 0;
      for (int q = 0; q < tid; ++q) rank += cid[q] == e;
      order[base[e] + rank] = i;
    }
    __syncthreads();
    if (e >= 0) atomicAdd(&base[e], 1);
    __syncthreads();
  }
}

// The same plan for up to 48 experts, without the walk over each chunk: thread t owns the run of pairs
// [t L, (t + 1) L), counts them by expert into cnt[t][e] (LDS), thread e then turns column e into each run's first
// place, and every thread puts its run's pairs there in order.
__global__ __launch_bounds__(256) void plan_runs_kernel(const int* ids, int n, int E, int* offsets, int* order) {
  extern __shared__ int cnt[];      // [256][E]
  const int tid = threadIdx.x;
  const int R = min(256, (n + 3) / 4);      // runs: four pairs a thread at least, so that few pairs make a short scan
  const int L = (n + R - 1) / R, lo = min(tid * L, n), hi = min(lo + L, n);
  if (tid < R)
    for (int e = 0; e < E; ++e) cnt[tid * E + e] = 0;
  for (int i = lo; i < hi; ++i) cnt[tid * E + ids[i]] += 1;
  __syncthreads();
  __shared__ int total[49];
  if (tid < E) {
    int run = 0;
    for (int t = 0; t < R; ++t) {
      const int c = cnt[t * E + tid];
      cnt[t * E + tid] = run;
      run += c;
    }
    total[tid] = run;
  }
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = run;
      run += total[e];
    }
    offsets[E] = run;
    for (int e = 0; e < E; ++e) total[e] = offsets[e];
  }
  __syncthreads();
  for (int i = lo; i < hi; ++i) {
    const int e = ids[i];
    order[total[e] + cnt[tid * E + e]++] = i;
  }
}

// which expert and which of its tiles of 16 places workgroup `id` has; false: none
__device__ __forceinline__ bool expert_tile(const int* offsets, int E, int id, int& e, int& p0, int& p1) {
  for (e = 0; e < E; ++e) {
    const int cnt = offsets[e + 1] - offsets[e];
    const int tiles = (cnt + TM - 1) / TM;
    if (id < tiles) {
      p0 = offsets[e] + id * TM;
      p1 = min(p0 + TM, offsets[e + 1]);
      return true;
    }
    id -= tiles;
  }
  return false;
}

// ---- an expert's first half: y[p, :] = act(W_gate h, W_up h) ---------------------------------------------------
// kind 0: g * sigmoid(alpha g) * (u + 1) with g = min(W_gate h, limit), u = clamp(W_up h, +-limit)
// kind 1: silu(s g) * (s u), s the pair's own factor (in_scale[pair]; none: 1): the expert reads s h, and both products
//         are linear in what they read
// kind 2: relu(s u)^2: an expert without a gate; the kernels are then built without the second product (DUAL false)
struct ExpertAct {
  float limit, alpha;
  int kind;
  const float* in_scale;
};

__device__ __forceinline__ float expert_act(const ExpertAct& a, float g, float u, float s) {
  if (a.kind == 1) {
    const float gs = g * s;
    return gs / (1.0f + expf(-gs)) * (u * s);
  }
  if (a.kind == 2) {      // (no gate: g is not computed)
    const float r = fmaxf(u * s, 0.f);
    return r * r;
  }
  const float gv = fminf(g, a.limit), uv = fminf(fmaxf(u, -a.limit), a.limit);
  return gv / (1.0f + expf(-a.alpha * gv)) * (uv + 1.0f);
}

template <bool DUAL>
__global__ __launch_bounds__(256) void expert_up_kernel(const void* h, int h_dt, size_t ldh, const int* order, const int* offsets,
                                                        int E, int top, const void* wg, const void* wu, int w_dt, int ff, int width,
                                                        ExpertAct act, void* y, int y_dt) {
  __shared__ Tile lds, lds2;
  int e, p0, p1;
  if (!expert_tile(offsets, E, blockIdx.x, e, p0, p1)) return;
  const int tid = threadIdx.x, n0 = blockIdx.y * TN;
  long long a_row[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int p = p0 + (tid >> 5) + 8 * q;
    a_row[q] = p < p1 ? static_cast<long long>(order[p] / top) * ldh : -1;
  }
  float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
  if (DUAL) tile_product<true>(lds, &lds2, h, h_dt, a_row, wg, wu, w_dt, static_cast<size_t>(e) * ff * width, ff, width, n0, g, u);
  else tile_product<false>(lds, nullptr, h, h_dt, a_row, wu, nullptr, w_dt, static_cast<size_t>(e) * ff * width, ff, width, n0, u, nullptr);
  const int p = p0 + (tid >> 4);
  if (p >= p1) return;
  const float sc = act.in_scale ? act.in_scale[order[p]] : 1.0f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int n = n0 + (tid & 15) * 4 + c;
    if (n >= ff) continue;
    store_as(y, static_cast<size_t>(p) * ff + n, y_dt, expert_act(act, g[c], u[c], sc));
  }
}

// ---- an expert's second half: out[pair, :] = W_down y[p, :] ------------------------------------------------------
__global__ __launch_bounds__(256) void expert_down_kernel(const void* y, int y_dt, const int* order, const int* offsets, int E,
                                                          const void* wd, int w_dt, int width, int ff, float* out) {
  __shared__ Tile lds;
  int e, p0, p1;
  if (!expert_tile(offsets, E, blockIdx.x, e, p0, p1)) return;
  const int tid = threadIdx.x, n0 = blockIdx.y * TN;
  long long a_row[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int p = p0 + (tid >> 5) + 8 * q;
    a_row[q] = p < p1 ? static_cast<long long>(p) * ff : -1;
  }
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  tile_product<false>(lds, nullptr, y, y_dt, a_row, wd, nullptr, w_dt, static_cast<size_t>(e) * width * ff, width, ff, n0, acc, nullptr);
  const int p = p0 + (tid >> 4);
  if (p >= p1) return;
  const size_t pair = order[p];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int n = n0 + (tid & 15) * 4 + c;
    if (n < width) out[pair * width + n] = acc[c];
  }
}

// x[t, :] += sum_c wts[t, c] * out[t * top + c, :], the choices in their order (wts none: every weight is 1)
// (logits: a weight is sigmoid of what wts holds; the weights of a row are then ldw numbers apart)
__global__ __launch_bounds__(256) void combine_kernel(const float* out, const float* wts, size_t ldw, int logits, int top, int width,
                                                      float* x, size_t ldx) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += 256) {
    float acc = 0.f;
    for (int q = 0; q < top; ++q) {
      float wq = wts ? wts[t * ldw + q] : 1.0f;
      if (logits) wq = 1.0f / (1.0f + expf(-wq));
      acc = fmaf(wq, out[(static_cast<size_t>(t) * top + q) * width + c], acc);
    }
    x[t * ldx + c] += acc;
  }
}

// ---- the same products on the matrix cores (bfloat16) ------------------------------------------------------------
// A workgroup of four waves takes 64 rows x 64 columns, a wave 32 x 32 as 2 x 2 blocks of v_mfma_f32_16x16x32_bf16.
// Operands go from memory straight into the lanes that the instruction reads them from: lane l holds the 8 numbers
// from k = 8 (l / 16) of row (or column) l % 16, 16 bytes in one load, so a step of 32 along K is one load per block
// and lane, no LDS and no barrier; the waves of a workgroup share their rows and columns through the vector cache.
// A block's sums: lane l holds row l % 16, columns 4 (l / 16) .. + 3.  Rows beyond a tile's last are read from its
// last row and stored nowhere.  K is a multiple of 32; every row starts at a multiple of 16 bytes.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
constexpr int MT = 64;      // rows of a workgroup's tile

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

// acc[i][j] += A[rows i] . W[cols j]^T over K; a_ptr[i], w_ptr[j]: this lane's row of block i / column of block j, at
// its own k offset.  PACKED: W lies in blocks of 16 columns x 32 of K in the lanes' own order (dn_pack_matrix): w_ptr[j]
// is the lane's 16 bytes of the column block's first step, a step further 512 numbers on; a load is then 1 KB in one
// piece, where from rows it touches 16 cache lines per 16 lanes, and the rate of those lookups is what bounds the kernel.
template <bool DUAL, bool PACKED, int CB>
__device__ __forceinline__ void mfma_tile(const bf16_t* const a_ptr[2], const bf16_t* const w_ptr[CB], const bf16_t* const w2_ptr[CB],
                                          int K, f32x4 acc[2][CB], f32x4 acc2[2][CB]) {
  constexpr int WSTEP = PACKED ? 512 : 32;
#pragma unroll 2
  for (int k0 = 0; k0 < K; k0 += 32) {
    bf16x8 af[2], wf[CB], wf2[CB];
#pragma unroll
    for (int i = 0; i < 2; ++i) af[i] = load8(a_ptr[i] + k0);
#pragma unroll
    for (int j = 0; j < CB; ++j) {
      wf[j] = load8(w_ptr[j] + static_cast<size_t>(k0 / 32) * WSTEP);
      if (DUAL) wf2[j] = load8(w2_ptr[j] + static_cast<size_t>(k0 / 32) * WSTEP);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < CB; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], af[i], acc[i][j], 0, 0, 0);
        if (DUAL) acc2[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf2[j], af[i], acc2[i][j], 0, 0, 0);
      }
  }
}

// The same with packed W and rows that are gathered (a token's row per pair): a lane asks for the 16 bytes `chunk = l % 4`
// of row l / 4, so that four neighbouring lanes read one row's 64 bytes (a load then touches 16 cache lines, not 64), and
// the block goes through a piece of LDS of the wave's own to the lanes that the instruction wants it in (lane l: row
// l % 16, chunk l / 16).  A wave's LDS accesses run in the order asked, so no barrier stands between the two.
template <bool DUAL, int CB>
__device__ __forceinline__ void mfma_tile_staged(bf16x8* stage, const bf16_t* const a_src[2], const bf16_t* const w_ptr[CB],
                                                 const bf16_t* const w2_ptr[CB], int K, f32x4 acc[2][CB], f32x4 acc2[2][CB]) {
  const int lane = threadIdx.x & 63;
  const int put = (lane & 3) * 16 + (lane >> 2);
#pragma unroll 2
  for (int k0 = 0; k0 < K; k0 += 32) {
    bf16x8 af[2], wf[CB], wf2[CB];
#pragma unroll
    for (int i = 0; i < 2; ++i) stage[i * 64 + put] = load8(a_src[i] + k0);
#pragma unroll
    for (int j = 0; j < CB; ++j) {
      wf[j] = load8(w_ptr[j] + static_cast<size_t>(k0 / 32) * 512);
      if (DUAL) wf2[j] = load8(w2_ptr[j] + static_cast<size_t>(k0 / 32) * 512);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) af[i] = stage[i * 64 + lane];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < CB; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], af[i], acc[i][j], 0, 0, 0);
        if (DUAL) acc2[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf2[j], af[i], acc2[i][j], 0, 0, 0);
      }
  }
}

// Workgroups are handed to the eight XCDs in turn, and each XCD has an L2 of its own: the launch is one line of
// workgroups, and workgroup L takes the work L' = (L % 8) * (n / 8) + L / 8, so that an XCD gets a run of neighbouring
// tiles (row tiles fastest: the tiles of one expert and column block, which read the same weights, meet in one L2).
// n: the launch's size, a multiple of 8; -> (row tile, column tile), or row tile -1 beyond `tiles_x * tiles_y`.
__device__ __forceinline__ void xcd_tile(int tiles_x, int tiles_y, int& tx, int& ty) {
  const int n = gridDim.x, L = blockIdx.x;
  const int at = (L % 8) * (n / 8) + L / 8;
  tx = at < tiles_x * tiles_y ? at % tiles_x : -1;
  ty = at / tiles_x;
}

// which expert and which of its tiles of 64 places workgroup `id` has.  The experts' offsets come to LDS in one
// parallel load first (a walk through them in memory is a chain of dependent loads, as long as the tile's own work).
constexpr int OFFSETS_IN_LDS = 1024;
__device__ __forceinline__ bool expert_tile64(const int* offsets, int E, int id, int& e, int& p0, int& p1) {
  __shared__ int held[OFFSETS_IN_LDS + 1];
  const bool in_lds = E <= OFFSETS_IN_LDS;
  if (in_lds) {
    for (int i = threadIdx.x; i <= E; i += blockDim.x) held[i] = offsets[i];
    __syncthreads();
  }
  const int* off = in_lds ? held : offsets;
  for (e = 0; e < E; ++e) {
    const int cnt = off[e + 1] - off[e];
    const int tiles = (cnt + MT - 1) / MT;
    if (id < tiles) {
      p0 = off[e] + id * MT;
      p1 = min(p0 + MT, off[e + 1]);
      return true;
    }
    id -= tiles;
  }
  return false;
}

template <bool DUAL>
__global__ __launch_bounds__(256) void expert_up_mfma_kernel(const bf16_t* h, size_t ldh, const int* order, const int* offsets, int E,
                                                             int top, const bf16_t* wg, const bf16_t* wu, int ff, int width,
                                                             ExpertAct act, bf16_t* y, int tiles_x) {
  int e, p0, p1, tx, ty;
  xcd_tile(tiles_x, (ff + 63) / 64, tx, ty);
  if (tx < 0 || !expert_tile64(offsets, E, tx, e, p0, p1)) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pw = p0 + (wave >> 1) * 32, nw = ty * 64 + (wave & 1) * 32;
  if (pw >= p1 || nw >= ff) return;
  const int kq = (lane >> 4) * 8, lr = lane & 15;
  const bf16_t *a_ptr[2], *g_ptr[2], *u_ptr[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int p = min(pw + 16 * i + lr, p1 - 1);
    a_ptr[i] = h + static_cast<size_t>(order[p] / top) * ldh + kq;
    const size_t n = min(nw + 16 * i + lr, ff - 1);
    g_ptr[i] = DUAL ? wg + (static_cast<size_t>(e) * ff + n) * width + kq : nullptr;
    u_ptr[i] = wu + (static_cast<size_t>(e) * ff + n) * width + kq;
  }
  f32x4 g[2][2] = {}, u[2][2] = {};
  if (DUAL) mfma_tile<true, false, 2>(a_ptr, g_ptr, u_ptr, width, g, u);
  else mfma_tile<false, false, 2>(a_ptr, u_ptr, nullptr, width, u, nullptr);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int p = pw + 16 * i + lr;
    if (p >= p1) continue;
    const float sc = act.in_scale ? act.in_scale[order[p]] : 1.0f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = nw + 16 * j + (lane >> 4) * 4;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (n + r >= ff) continue;
        y[static_cast<size_t>(p) * ff + n + r] = from_float<bf16_t>(expert_act(act, g[i][j][r], u[i][j][r], sc));
      }
    }
  }
}

__global__ __launch_bounds__(256) void expert_down_mfma_kernel(const bf16_t* y, const int* order, const int* offsets, int E,
                                                               const bf16_t* wd, int width, int ff, float* out, int tiles_x) {
  int e, p0, p1, tx, ty;
  xcd_tile(tiles_x, (width + 63) / 64, tx, ty);
  if (tx < 0 || !expert_tile64(offsets, E, tx, e, p0, p1)) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pw = p0 + (wave >> 1) * 32, nw = ty * 64 + (wave & 1) * 32;
  if (pw >= p1 || nw >= width) return;
  const int kq = (lane >> 4) * 8, lr = lane & 15;
  const bf16_t *a_ptr[2], *w_ptr[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    a_ptr[i] = y + static_cast<size_t>(min(pw + 16 * i + lr, p1 - 1)) * ff + kq;
    w_ptr[i] = wd + (static_cast<size_t>(e) * width + min(nw + 16 * i + lr, width - 1)) * ff + kq;
  }
  f32x4 acc[2][2] = {};
  mfma_tile<false, false, 2>(a_ptr, w_ptr, nullptr, ff, acc, nullptr);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int p = pw + 16 * i + lr;
    if (p >= p1) continue;
    const size_t pair = order[p];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = nw + 16 * j + (lane >> 4) * 4;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < width) out[pair * width + n + r] = acc[i][j][r];
    }
  }
}


// The same two kernels for packed weights (the experts' matrices stacked and packed as one; an expert's rows start at a
// multiple of 16): a wave takes 32 pairs x 64 columns, a workgroup 64 x 128; where the step has few pairs an expert
// (decoded tokens: the kernel then only streams the chosen experts' matrices) a wave takes 16 columns, so that four
// times as many waves have loads in flight.  An element's sum is the same in both.
template <int CB, bool DUAL>
__global__ __launch_bounds__(256) void expert_up_packed_kernel(const bf16_t* h, size_t ldh, const int* order, const int* offsets, int E,
                                                               int top, const bf16_t* wg, const bf16_t* wu, int ff, int width,
                                                               ExpertAct act, bf16_t* y, int tiles_x) {
  int e, p0, p1, tx, ty;
  xcd_tile(tiles_x, (ff + 32 * CB - 1) / (32 * CB), tx, ty);
  if (tx < 0 || !expert_tile64(offsets, E, tx, e, p0, p1)) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pw = p0 + (wave >> 1) * 32, nw = ty * (32 * CB) + (wave & 1) * (16 * CB);
  if (pw >= p1 || nw >= ff) return;
  __shared__ bf16x8 stage[4][128];
  const int lr = lane & 15, ksteps = width / 32;
  const bf16_t *a_ptr[2], *g_ptr[CB], *u_ptr[CB];
#pragma unroll
  for (int i = 0; i < 2; ++i)
    a_ptr[i] = h + static_cast<size_t>(order[min(pw + 16 * i + (lane >> 2), p1 - 1)] / top) * ldh + (lane & 3) * 8;
#pragma unroll
  for (int j = 0; j < CB; ++j) {
    const size_t block = (static_cast<size_t>(e) * ff + min(nw + 16 * j, ff - 16)) / 16;
    g_ptr[j] = DUAL ? wg + block * ksteps * 512 + lane * 8 : nullptr;
    u_ptr[j] = wu + block * ksteps * 512 + lane * 8;
  }
  f32x4 g[2][CB] = {}, u[2][CB] = {};
  if (DUAL) mfma_tile_staged<true, CB>(stage[wave], a_ptr, g_ptr, u_ptr, width, g, u);
  else mfma_tile_staged<false, CB>(stage[wave], a_ptr, u_ptr, nullptr, width, u, nullptr);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int p = pw + 16 * i + lr;
    if (p >= p1) continue;
    const float sc = act.in_scale ? act.in_scale[order[p]] : 1.0f;
#pragma unroll
    for (int j = 0; j < CB; ++j) {
      const int n = nw + 16 * j + (lane >> 4) * 4;
      if (n >= ff) continue;      // (ff is a multiple of 16: a block is whole or absent)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        y[static_cast<size_t>(p) * ff + n + r] = from_float<bf16_t>(expert_act(act, g[i][j][r], u[i][j][r], sc));
    }
  }
}

template <int CB>
__global__ __launch_bounds__(256) void expert_down_packed_kernel(const bf16_t* y, const int* order, const int* offsets, int E,
                                                                 const bf16_t* wd, int width, int ff, float* out, int tiles_x) {
  int e, p0, p1, tx, ty;
  xcd_tile(tiles_x, (width + 32 * CB - 1) / (32 * CB), tx, ty);
  if (tx < 0 || !expert_tile64(offsets, E, tx, e, p0, p1)) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pw = p0 + (wave >> 1) * 32, nw = ty * (32 * CB) + (wave & 1) * (16 * CB);
  if (pw >= p1 || nw >= width) return;
  __shared__ bf16x8 stage[4][128];
  const int lr = lane & 15, ksteps = ff / 32;
  const bf16_t *a_ptr[2], *w_ptr[CB];
#pragma unroll
  for (int i = 0; i < 2; ++i) a_ptr[i] = y + static_cast<size_t>(min(pw + 16 * i + (lane >> 2), p1 - 1)) * ff + (lane & 3) * 8;
#pragma unroll
  for (int j = 0; j < CB; ++j)
    w_ptr[j] = wd + (static_cast<size_t>(e) * width + min(nw + 16 * j, width - 16)) / 16 * ksteps * 512 + lane * 8;
  f32x4 acc[2][CB] = {};
  mfma_tile_staged<false, CB>(stage[wave], a_ptr, w_ptr, nullptr, ff, acc, nullptr);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int p = pw + 16 * i + lr;
    if (p >= p1) continue;
    const size_t pair = order[p];
#pragma unroll
    for (int j = 0; j < CB; ++j) {
      const int n = nw + 16 * j + (lane >> 4) * 4;
      if (n >= width) continue;
      *reinterpret_cast<f32x4*>(out + pair * width + n) = acc[i][j];
    }
  }
}

// out[t, o_off + h * o_stride + n] = sum_k W[h][n][k] a[t, a_off + h * a_stride + k] on the matrix cores, 32-bit sums.
// AF32: the rows are 32-bit and are rounded to bfloat16 on their way into the instruction (two loads of 16 bytes a lane
// and step in place of one).
template <bool AF32>
__global__ __launch_bounds__(256) void heads_linear_mfma_kernel(const void* A, size_t lda, int a_off, int a_stride, const bf16_t* W,
                                                                void* out, int out_dt, size_t ldo, int o_off, int o_stride, int T,
                                                                int N, int K) {
  const int hd = blockIdx.z, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tw = blockIdx.x * MT + (wave >> 1) * 32, nw = blockIdx.y * 64 + (wave & 1) * 32;
  if (tw >= T || nw >= N) return;
  const int kq = (lane >> 4) * 8, lr = lane & 15;
  size_t a_at[2];
  const bf16_t* w_ptr[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    a_at[i] = static_cast<size_t>(min(tw + 16 * i + lr, T - 1)) * lda + a_off + static_cast<size_t>(hd) * a_stride + kq;
    w_ptr[i] = W + (static_cast<size_t>(hd) * N + min(nw + 16 * i + lr, N - 1)) * K + kq;
  }
  f32x4 acc[2][2] = {};
#pragma unroll 2
  for (int k0 = 0; k0 < K; k0 += 32) {
    bf16x8 af[2], wf[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if constexpr (AF32) {
        const float* p = static_cast<const float*>(A) + a_at[i] + k0;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(p), hi = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) af[i][e] = static_cast<__bf16>(lo[e]), af[i][4 + e] = static_cast<__bf16>(hi[e]);
      } else {
        af[i] = load8(static_cast<const bf16_t*>(A) + a_at[i] + k0);
      }
      wf[i] = load8(w_ptr[i] + k0);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], af[i], acc[i][j], 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int t = tw + 16 * i + lr;
    if (t >= T) continue;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = nw + 16 * j + (lane >> 4) * 4;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < N) store_as(out, static_cast<size_t>(t) * ldo + o_off + static_cast<size_t>(hd) * o_stride + n + r, out_dt, acc[i][j][r]);
    }
  }
}

bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

bool float_kind(int dt) { return dt == DN_F32 || dt == DN_BF16; }

}  // namespace

extern "C" {

int dn_heads_linear(const void* a, int a_dt, long long lda, int a_off, int a_stride, const void* w, int w_dt, void* out, int out_dt,
                    long long ldo, int o_off, int o_stride, int T, int H, int N, int K, hipStream_t stream) {
  if (!float_kind(a_dt) || !float_kind(w_dt) || !float_kind(out_dt)) return DN_ERR_DTYPE;
  if (H < 1 || N < 1 || K < 1 || H > 65535) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  // bfloat16 weights take the matrix cores; 32-bit rows are rounded to bfloat16 on the way in, but only where the result
  // is bfloat16 too (a 32-bit result of 32-bit rows keeps the vector kernel's 32-bit products)
  const int per16 = a_dt == DN_BF16 ? 8 : 4;
  if (w_dt == DN_BF16 && (a_dt == DN_BF16 || out_dt == DN_BF16) && K % 32 == 0 && lda % per16 == 0 && a_off % per16 == 0 &&
      a_stride % per16 == 0 && aligned16(a) && aligned16(w)) {
    const dim3 grid((T + MT - 1) / MT, (N + 63) / 64, H);
    if (a_dt == DN_BF16)
      hipLaunchKernelGGL(heads_linear_mfma_kernel<false>, grid, dim3(256), 0, stream, a, static_cast<size_t>(lda), a_off, a_stride,
                         static_cast<const bf16_t*>(w), out, out_dt, static_cast<size_t>(ldo), o_off, o_stride, T, N, K);
    else
      hipLaunchKernelGGL(heads_linear_mfma_kernel<true>, grid, dim3(256), 0, stream, a, static_cast<size_t>(lda), a_off, a_stride,
                         static_cast<const bf16_t*>(w), out, out_dt, static_cast<size_t>(ldo), o_off, o_stride, T, N, K);
    return dn_launch_status();
  }
  hipLaunchKernelGGL(heads_linear_kernel, dim3((T + TM - 1) / TM, (N + TN - 1) / TN, H), dim3(256), 0, stream, a, a_dt,
                     static_cast<size_t>(lda), a_off, a_stride, w, w_dt, out, out_dt, static_cast<size_t>(ldo), o_off, o_stride, T, N, K);
  return dn_launch_status();
}

int dn_moe_route(const float* z, long long ldz, const float* correction, int T, int E, int top, int sigmoid, int renorm, int* ids,
                 float* wts, int groups, int keep, float scale, hipStream_t stream) {
  if (E < 1 || top < 1 || top > E || ldz < E) return DN_ERR_SHAPE;
  if (groups < 1 || E % groups != 0 || keep < 1 || keep > groups || top > keep * (E / groups)) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  if (E <= 8192 && top <= 64) {
    hipLaunchKernelGGL(route_wave_kernel, dim3(T), dim3(64), 0, stream, z, static_cast<size_t>(ldz), correction, E, top, sigmoid, renorm,
                       ids, wts, keep < groups ? groups : 1, keep, scale);
    return dn_launch_status();
  }
  if (keep < groups || scale != 1.0f) return DN_ERR_SHAPE;      // (the kernel of a thread a row knows neither)
  hipLaunchKernelGGL(route_kernel, dim3((T + 63) / 64), dim3(64), 0, stream, z, static_cast<size_t>(ldz), correction, T, E, top, sigmoid,
                     renorm, ids, wts);
  return dn_launch_status();
}

int dn_moe_plan(const int* ids, int n, int E, int* offsets, int* order, hipStream_t stream) {
  if (E < 1 || E > 8192) return DN_ERR_SHAPE;
  if (E <= 48)
    hipLaunchKernelGGL(plan_runs_kernel, dim3(1), dim3(256), 256 * E * sizeof(int), stream, ids, n, E, offsets, order);
  else
    hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(256), (E + 256) * sizeof(int), stream, ids, n, E, offsets, order);
  return dn_launch_status();
}

int dn_moe_up(const void* h, int h_dt, long long ldh, const int* order, const int* offsets, int E, int top, int n, const void* wg,
              const void* wu, int w_dt, int ff, int width, float limit, float alpha, int kind, const float* in_scale, void* y,
              int y_dt, int packed, hipStream_t stream) {
  if (!float_kind(h_dt) || !float_kind(w_dt) || !float_kind(y_dt)) return DN_ERR_DTYPE;
  if (kind < 0 || kind > 2) return DN_ERR_SHAPE;
  const bool dual = kind != 2;
  if (n == 0) return 0;
  const ExpertAct act{limit, alpha, kind, in_scale};
  if (packed) {
    if (h_dt != DN_BF16 || w_dt != DN_BF16 || y_dt != DN_BF16) return DN_ERR_DTYPE;
    if (width % 32 != 0 || ff % 16 != 0 || ldh % 8 != 0 || !aligned16(h) || (dual && !aligned16(wg)) || !aligned16(wu)) return DN_ERR_SHAPE;
    const int tiles_x = (n + MT - 1) / MT + E;
    if (n <= 16 * E) {
      const int tiles = tiles_x * ((ff + 31) / 32);
      if (dual) hipLaunchKernelGGL((expert_up_packed_kernel<1, true>), dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream, static_cast<const bf16_t*>(h),
                         static_cast<size_t>(ldh), order, offsets, E, top, static_cast<const bf16_t*>(wg),
                         static_cast<const bf16_t*>(wu), ff, width, act, static_cast<bf16_t*>(y), tiles_x);
      else hipLaunchKernelGGL((expert_up_packed_kernel<1, false>), dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream, static_cast<const bf16_t*>(h),
                         static_cast<size_t>(ldh), order, offsets, E, top, static_cast<const bf16_t*>(wg),
                         static_cast<const bf16_t*>(wu), ff, width, act, static_cast<bf16_t*>(y), tiles_x);
    } else {
      const int tiles = tiles_x * ((ff + 127) / 128);
      if (dual) hipLaunchKernelGGL((expert_up_packed_kernel<4, true>), dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream, static_cast<const bf16_t*>(h),
                         static_cast<size_t>(ldh), order, offsets, E, top, static_cast<const bf16_t*>(wg),
                         static_cast<const bf16_t*>(wu), ff, width, act, static_cast<bf16_t*>(y), tiles_x);
      else hipLaunchKernelGGL((expert_up_packed_kernel<4, false>), dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream, static_cast<const bf16_t*>(h),
                         static_cast<size_t>(ldh), order, offsets, E, top, static_cast<const bf16_t*>(wg),
                         static_cast<const bf16_t*>(wu), ff, width, act, static_cast<bf16_t*>(y), tiles_x);
    }
    return dn_launch_status();
  }
  if (h_dt == DN_BF16 && w_dt == DN_BF16 && y_dt == DN_BF16 && width % 32 == 0 && ldh % 8 == 0 && aligned16(h) && (!dual || aligned16(wg)) &&
      aligned16(wu)) {
    const int tiles_x = (n + MT - 1) / MT + E, tiles = tiles_x * ((ff + 63) / 64);
    if (dual) hipLaunchKernelGGL(expert_up_mfma_kernel<true>, dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream,
                       static_cast<const bf16_t*>(h), static_cast<size_t>(ldh), order, offsets, E, top, static_cast<const bf16_t*>(wg),
                       static_cast<const bf16_t*>(wu), ff, width, act, static_cast<bf16_t*>(y), tiles_x);
  else hipLaunchKernelGGL(expert_up_mfma_kernel<false>, dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream,
                       static_cast<const bf16_t*>(h), static_cast<size_t>(ldh), order, offsets, E, top, static_cast<const bf16_t*>(wg),
                       static_cast<const bf16_t*>(wu), ff, width, act, static_cast<bf16_t*>(y), tiles_x);
    return dn_launch_status();
  }
  if (dual) hipLaunchKernelGGL(expert_up_kernel<true>, dim3((n + TM - 1) / TM + E, (ff + TN - 1) / TN), dim3(256), 0, stream, h, h_dt,
                     static_cast<size_t>(ldh), order, offsets, E, top, wg, wu, w_dt, ff, width, act, y, y_dt);
  else hipLaunchKernelGGL(expert_up_kernel<false>, dim3((n + TM - 1) / TM + E, (ff + TN - 1) / TN), dim3(256), 0, stream, h, h_dt,
                     static_cast<size_t>(ldh), order, offsets, E, top, wg, wu, w_dt, ff, width, act, y, y_dt);
  return dn_launch_status();
}

int dn_moe_down(const void* y, int y_dt, const int* order, const int* offsets, int E, int n, const void* wd, int w_dt, int width,
                int ff, float* out, int packed, hipStream_t stream) {
  if (!float_kind(y_dt) || !float_kind(w_dt)) return DN_ERR_DTYPE;
  if (n == 0) return 0;
  if (packed) {
    if (y_dt != DN_BF16 || w_dt != DN_BF16) return DN_ERR_DTYPE;
    if (ff % 32 != 0 || width % 16 != 0 || !aligned16(y) || !aligned16(wd) || !aligned16(out)) return DN_ERR_SHAPE;
    const int tiles_x = (n + MT - 1) / MT + E;
    if (n <= 16 * E) {
      const int tiles = tiles_x * ((width + 31) / 32);
      hipLaunchKernelGGL(expert_down_packed_kernel<1>, dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream, static_cast<const bf16_t*>(y),
                         order, offsets, E, static_cast<const bf16_t*>(wd), width, ff, out, tiles_x);
    } else {
      const int tiles = tiles_x * ((width + 127) / 128);
      hipLaunchKernelGGL(expert_down_packed_kernel<4>, dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream, static_cast<const bf16_t*>(y),
                         order, offsets, E, static_cast<const bf16_t*>(wd), width, ff, out, tiles_x);
    }
    return dn_launch_status();
  }
  if (y_dt == DN_BF16 && w_dt == DN_BF16 && ff % 32 == 0 && aligned16(y) && aligned16(wd)) {
    const int tiles_x = (n + MT - 1) / MT + E, tiles = tiles_x * ((width + 63) / 64);
    hipLaunchKernelGGL(expert_down_mfma_kernel, dim3((tiles + 7) / 8 * 8), dim3(256), 0, stream,
                       static_cast<const bf16_t*>(y), order, offsets, E, static_cast<const bf16_t*>(wd), width, ff, out, tiles_x);
    return dn_launch_status();
  }
  hipLaunchKernelGGL(expert_down_kernel, dim3((n + TM - 1) / TM + E, (width + TN - 1) / TN), dim3(256), 0, stream, y, y_dt, order,
                     offsets, E, wd, w_dt, width, ff, out);
  return dn_launch_status();
}

int dn_moe_combine(const float* out, const float* wts, long long ldw, int logits, int T, int top, int width, float* x, long long ldx,
                   hipStream_t stream) {
  if (T == 0) return 0;
  hipLaunchKernelGGL(combine_kernel, dim3(T), dim3(256), 0, stream, out, wts, static_cast<size_t>(ldw), logits, top, width, x,
                     static_cast<size_t>(ldx));
  return dn_launch_status();
}

}  // extern "C"
