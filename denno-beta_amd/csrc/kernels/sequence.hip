// Kernels for layers that carry something from token to token besides keys and values: norms without a
// mean, short causal convolutions over time, the previous token's row, turned pairs of dimensions, and
// matrix states that decay (one scan for every recurrence of the form S <- diag(w) S + a v^T, and for the delta rule,
// which writes what the state does not yet answer to a key), norms that add into the stream, averages over depth.
// Everything here is 32-bit arithmetic; only what is read or stored may be bfloat16.  A request's rows
// are rows row_start[s] .. row_start[s + 1] - 1 of the step, its state lies at slots[s]; a request whose
// slot is negative is padding and is skipped.
#include "common.h"

namespace {

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

__device__ __forceinline__ float load_as(const void* p, size_t i, int dt) {
  return dt == DN_F32 ? static_cast<const float*>(p)[i] : to_float(static_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void store_as(void* p, size_t i, int dt, float v) {
  if (dt == DN_F32) static_cast<float*>(p)[i] = v;
  else static_cast<bf16_t*>(p)[i] = from_float<bf16_t>(v);
}

// the request that owns row t: the last s with row_start[s] <= t
__device__ __forceinline__ int request_of(const int* row_start, int S, int t) {
  int lo = 0, hi = S - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (row_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// sum over a workgroup of 256 threads, the same in every thread; waves are joined in order
__device__ __forceinline__ float block_sum_256(float v, float* sh) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh[wave] = v;
  __syncthreads();
  return (sh[0] + sh[1]) + (sh[2] + sh[3]);
}

// ---- norm without a mean -----------------------------------------------------------------------------------
// out[r, :] = x[row, :width] / sqrt(mean(x^2) + eps) * weight; one workgroup a row; a thread sums its own
// columns in ascending order, so a row's result does not depend on what else is in the step.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const void* x, int x_dt, size_t ldx, const float* weight, void* out,
                                                      int out_dt, size_t ldo, const int* rows, int width, float eps) {
  __shared__ float sh[4];
  const int r = blockIdx.x;
  const size_t src = static_cast<size_t>(rows ? rows[r] : r) * ldx;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = load_as(x, src + c, x_dt);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum_256(ss, sh);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(width) + eps);
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = load_as(x, src + c, x_dt) * inv;
    store_as(out, static_cast<size_t>(r) * ldo + c, out_dt, weight ? v * weight[c] : v);
  }
}

// x[t, :] += mult * (y[t, :] / sqrt(mean(y^2) + eps) * weight) * scale: the norm of a sublayer's result, added into the
// stream (scale: a vector, or none).  gate: y is y * sigmoid(gate[t, :]) first, under the norm's sums too (a gate on the
// sublayer's result).  next_out: the row as it then stands, normed for whoever reads the stream next (next_w, next_eps): a
// launch less between two sublayers.  One workgroup a row, the sums as in rmsnorm_kernel.
__global__ __launch_bounds__(256) void rmsnorm_add_kernel(const void* y, int y_dt, size_t ldy, const float* weight, const float* scale,
                                                          float mult, float* x, size_t ldx, int width, float eps, const float* gate,
                                                          size_t ldg, const float* next_w, float next_eps, void* next_out, int next_dt,
                                                          size_t ldn) {
  __shared__ float sh[4];
  const size_t src = static_cast<size_t>(blockIdx.x) * ldy, dst = static_cast<size_t>(blockIdx.x) * ldx;
  const float* g = gate ? gate + static_cast<size_t>(blockIdx.x) * ldg : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    float v = load_as(y, src + c, y_dt);
    if (g) v *= 1.0f / (1.0f + expf(-g[c]));
    ss = fmaf(v, v, ss);
  }
  ss = block_sum_256(ss, sh);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(width) + eps);
  float after = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    float v = load_as(y, src + c, y_dt);
    if (g) v *= 1.0f / (1.0f + expf(-g[c]));
    v *= inv;
    if (weight) v *= weight[c];
    if (scale) v *= scale[c];
    const float sum = fmaf(mult, v, x[dst + c]);
    x[dst + c] = sum;
    after = fmaf(sum, sum, after);
  }
  if (!next_out) return;
  // the norm that reads the stream next, on the row as it stands now: the sums as rmsnorm_kernel makes them (the same bits)
  after = block_sum_256(after, sh);
  const float inv2 = 1.0f / sqrtf(after / static_cast<float>(width) + next_eps);
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = x[dst + c] * inv2;      // (the thread's own store)
    store_as(next_out, static_cast<size_t>(blockIdx.x) * ldn + c, next_dt, next_w ? v * next_w[c] : v);
  }
}

// out[i] = sum_j w[j] * hist[j][i], j ascending from 0 to n - 1, one fused multiply-add a step: an average over the
// streams that the layers so far have left ([n][rows * width], `plane` numbers apart).  out may be a later plane.
__global__ __launch_bounds__(256) void depth_mix_kernel(const float* hist, size_t plane, int n, const float* w, float* out, size_t total,
                                                        int vec) {
  const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i >= total) return;
  if (vec && i + 4 <= total) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < n; ++j) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(hist + j * plane + i);
      const float wj = w[j];
      acc[0] = fmaf(wj, v[0], acc[0]), acc[1] = fmaf(wj, v[1], acc[1]), acc[2] = fmaf(wj, v[2], acc[2]), acc[3] = fmaf(wj, v[3], acc[3]);
    }
    *reinterpret_cast<f32x4*>(out + i) = acc;
  } else {
    for (size_t e = i; e < total && e < i + 4; ++e) {
      float acc = 0.f;
      for (int j = 0; j < n; ++j) acc = fmaf(w[j], hist[j * plane + e], acc);
      out[e] = acc;
    }
  }
}

// out[t, :] = [a[t, :wa] | b[t, :wb]]
__global__ __launch_bounds__(256) void concat_kernel(const float* a, size_t lda, int wa, const float* b, size_t ldb, int wb,
                                                     void* out, int out_dt) {
  const int t = blockIdx.x;
  const size_t o = static_cast<size_t>(t) * (wa + wb);
  for (int c = threadIdx.x; c < wa + wb; c += 256)
    store_as(out, o + c, out_dt, c < wa ? a[t * lda + c] : b[t * ldb + (c - wa)]);
}

// ---- short causal convolution over time ----------------------------------------------------------------------
// out[t, c] = act((identity ? h[t, c] : 0) + sum_j w[c, j] * h[t - taps + 1 + j, c]); rows before the step's first row of a
// request come from its history [slot][taps - 1][width] (oldest first; zero for a new request).  h and out are rows
// ldh and ldo numbers apart (the channels may be the first columns of wider rows); act: none or silu; bias: a number per
// channel that the sum starts from, or none.
__global__ __launch_bounds__(256) void conv_rows_kernel(const float* h, size_t ldh, const float* w, const float* bias, const float* hist, const int* row_start,
                                                        const int* slots, int S, int width, int taps, int identity, int silu, void* out,
                                                        int out_dt, size_t ldo, size_t hist_stride) {
  const int t = blockIdx.x;
  const int s = request_of(row_start, S, t);
  const int slot = slots[s];
  // (a row's channels are shared out among the workgroups of the grid's second dimension, 256 at a time)
  const int c0 = blockIdx.y * 256 + threadIdx.x, cstep = gridDim.y * 256;
  if (slot < 0 || t >= row_start[S]) {      // a padding row: zeros, so that what follows works on numbers
    for (int c = c0; c < width; c += cstep) store_as(out, static_cast<size_t>(t) * ldo + c, out_dt, 0.f);
    return;
  }
  const int i = t - row_start[s];
  const float* past = hist + static_cast<size_t>(slot) * hist_stride;
  for (int c = c0; c < width; c += cstep) {
    float acc = (identity ? h[static_cast<size_t>(t) * ldh + c] : 0.f) + (bias ? bias[c] : 0.f);
    for (int j = 0; j < taps; ++j) {
      const int src = i - taps + 1 + j;
      const float v = src >= 0 ? h[static_cast<size_t>(row_start[s] + src) * ldh + c] : past[static_cast<size_t>(i + j) * width + c];
      acc = fmaf(w[c * taps + j], v, acc);
    }
    if (silu) acc = acc / (1.0f + expf(-acc));
    store_as(out, static_cast<size_t>(t) * ldo + c, out_dt, acc);
  }
}

// The same convolution (without the row itself, then silu) over channels that are heads' vectors, a wave a vector, and for
// the vectors of the first `n_unit` heads (of `unit_dim` channels each; the others have `rest_dim`) the vector is then
// divided by sqrt(sum of its squares + eps) and multiplied by the head's scale: scale_a for the first n_a of them, scale_b
// for the others.  Queries, keys and values of a recurrence leave one kernel as the recurrence reads them.
__global__ __launch_bounds__(64) void conv_heads_kernel(const float* h, size_t ldh, const float* w, const float* hist, const int* row_start,
                                                        const int* slots, int S, int width, int taps, int n_unit, int unit_dim, int n_a,
                                                        float scale_a, float scale_b, float eps, int rest_dim, float* out, size_t ldo,
                                                        size_t hist_stride) {
  const int t = blockIdx.x, vec = blockIdx.y, lane = threadIdx.x;
  const bool unit = vec < n_unit;
  const int dim = unit ? unit_dim : rest_dim;
  const int c0 = unit ? vec * unit_dim : n_unit * unit_dim + (vec - n_unit) * rest_dim;
  float* dst = out + static_cast<size_t>(t) * ldo + c0;
  const int s = request_of(row_start, S, t);
  const int slot = slots[s];
  if (slot < 0 || t >= row_start[S]) {      // a padding row: zeros
    for (int j = lane; j < dim; j += 64) dst[j] = 0.f;
    return;
  }
  const int i = t - row_start[s];
  const float* past = hist + static_cast<size_t>(slot) * hist_stride;
  float ss = 0.f;
  for (int j = lane; j < dim; j += 64) {
    const int c = c0 + j;
    float acc = 0.f;
    for (int q = 0; q < taps; ++q) {
      const int src = i - taps + 1 + q;
      const float v = src >= 0 ? h[static_cast<size_t>(row_start[s] + src) * ldh + c] : past[static_cast<size_t>(i + q) * width + c];
      acc = fmaf(w[c * taps + q], v, acc);
    }
    acc = acc / (1.0f + expf(-acc));
    ss = fmaf(acc, acc, ss);
    dst[j] = acc;
  }
  if (!unit) return;
  ss = wave_sum(ss);
  const float f = (vec < n_a ? scale_a : scale_b) / sqrtf(ss + eps);
  for (int j = lane; j < dim; j += 64) dst[j] *= f;      // (a lane reads back what it wrote itself)
}

// The last `keep` rows of (history ++ this step's rows) become the history.  A thread owns a channel of a request and
// goes through the places in ascending order: place m reads the old place m + n, which it has not written yet.
__global__ __launch_bounds__(256) void history_update_kernel(const void* h, int h_dt, size_t ldh, float* hist, const int* row_start,
                                                             const int* slots, int width, int keep, size_t hist_stride) {
  const int s = blockIdx.x;
  const int slot = slots[s];
  if (slot < 0) return;
  const int row0 = row_start[s], n = row_start[s + 1] - row0;
  float* past = hist + static_cast<size_t>(slot) * hist_stride;
  for (int c = threadIdx.x; c < width; c += 256)
    for (int m = 0; m < keep; ++m) {
      const int src = n - keep + m;
      past[static_cast<size_t>(m) * width + c] =
          src >= 0 ? load_as(h, static_cast<size_t>(row0 + src) * ldh + c, h_dt) : past[static_cast<size_t>(m + n) * width + c];
    }
}

// out[m][t][c] = h[t][c] + (h[t - 1][c] - h[t][c]) * mu[m][c]; the row before a request's first row of the step is
// its history (one row a slot).
__global__ __launch_bounds__(256) void shift_mix_kernel(const void* h, int h_dt, const float* hist, const float* mu, int n_mix,
                                                        const int* row_start, const int* slots, int S, int T, int width,
                                                        void* out, int out_dt, size_t hist_stride) {
  const int t = blockIdx.x;
  const int s = request_of(row_start, S, t);
  const int slot = slots[s];
  if (slot < 0 || t >= row_start[S]) {      // a padding row
    for (int c = threadIdx.x; c < width; c += 256)
      for (int m = 0; m < n_mix; ++m) store_as(out, (static_cast<size_t>(m) * T + t) * width + c, out_dt, 0.f);
    return;
  }
  const bool first = t == row_start[s];
  for (int c = threadIdx.x; c < width; c += 256) {
    const float cur = load_as(h, static_cast<size_t>(t) * width + c, h_dt);
    const float prev = first ? hist[static_cast<size_t>(slot) * hist_stride + c] : load_as(h, static_cast<size_t>(t - 1) * width + c, h_dt);
    const float d = prev - cur;
    for (int m = 0; m < n_mix; ++m)
      store_as(out, (static_cast<size_t>(m) * T + t) * width + c, out_dt, fmaf(d, mu[m * width + c], cur));
  }
}

// ---- pairs of dimensions turned by the position ------------------------------------------------------------
// Vector n of row t starts at src_off + n * src_stride; its entries 2i and 2i + 1 (i < dims / 2) are turned by the
// angle position * freq[i] (cos and sin times `mag`: a scaled encoding's factor, 1 otherwise), the other `width - dims`
// entries pass; the result goes to dst_off + n * dst_stride.
__global__ __launch_bounds__(256) void rotary_kernel(const void* src, int src_dt, size_t ld_src, int src_off, int src_stride,
                                                     void* dst, int dst_dt, size_t ld_dst, int dst_off, int dst_stride,
                                                     const int* positions, const float* freq, int n_vec, int dims, int width,
                                                     float mag) {
  const int t = blockIdx.x;
  const float p = static_cast<float>(positions[t]);
  const int half = dims / 2, rest = width - dims;
  const int per = half + rest;
  for (int e = threadIdx.x; e < n_vec * per; e += 256) {
    const int n = e / per, i = e % per;
    const size_t a = static_cast<size_t>(t) * ld_src + src_off + static_cast<size_t>(n) * src_stride;
    const size_t b = static_cast<size_t>(t) * ld_dst + dst_off + static_cast<size_t>(n) * dst_stride;
    if (i < half) {
      const float ang = p * freq[i];
      const float c = cosf(ang) * mag, sn = sinf(ang) * mag;
      const float u = load_as(src, a + 2 * i, src_dt), v = load_as(src, a + 2 * i + 1, src_dt);
      store_as(dst, b + 2 * i, dst_dt, u * c - v * sn);
      store_as(dst, b + 2 * i + 1, dst_dt, v * c + u * sn);
    } else {
      const int k = dims + (i - half);
      store_as(dst, b + k, dst_dt, load_as(src, a + k, src_dt));
    }
  }
}

// Up to three runs of vectors of one row turned (or only moved) in one launch, each run to a place of its own: the
// queries, keys and values of a fused projection on their way to the attention's rows and the cache's.
struct TurnRun {
  void* dst;
  int dst_dt;
  size_t ld_dst;
  int src_off, dst_off, dst_stride, n_vec, width, dims;      // (src_stride is the width: the vectors lie side by side)
  int unit;      // the vectors are divided by their root mean square behind the turn (rotary_runs_unit_kernel)
};
struct TurnRuns {
  TurnRun run[3];
  int n;
};

__global__ __launch_bounds__(256) void rotary_runs_kernel(const void* src, int src_dt, size_t ld_src, TurnRuns runs, const int* positions,
                                                          const float* freq, float mag) {
  const int t = blockIdx.x;
  const float p = static_cast<float>(positions[t]);
  for (int r = 0; r < runs.n; ++r) {
    const TurnRun& u = runs.run[r];
    const int half = u.dims / 2, per = half + (u.width - u.dims);
    for (int e = threadIdx.x; e < u.n_vec * per; e += 256) {
      const int n = e / per, i = e % per;
      const size_t a = static_cast<size_t>(t) * ld_src + u.src_off + static_cast<size_t>(n) * u.width;
      const size_t b = static_cast<size_t>(t) * u.ld_dst + u.dst_off + static_cast<size_t>(n) * u.dst_stride;
      if (i < half) {
        const float ang = p * freq[i];
        const float c = cosf(ang) * mag, sn = sinf(ang) * mag;
        const float x = load_as(src, a + 2 * i, src_dt), y = load_as(src, a + 2 * i + 1, src_dt);
        store_as(u.dst, b + 2 * i, u.dst_dt, x * c - y * sn);
        store_as(u.dst, b + 2 * i + 1, u.dst_dt, y * c + x * sn);
      } else {
        const int k = u.dims + (i - half);
        store_as(u.dst, b + k, u.dst_dt, load_as(src, a + k, src_dt));
      }
    }
  }
}

// The same runs with a wave a vector (widths up to 256), for runs whose vectors are divided by their root mean square
// behind the turn (TurnRun.unit: x / sqrt(mean(x^2) + eps) over the vector's `width` entries): a lane holds the pairs
// lane and lane + 64 of its vector, the squares are summed over the wave in one order, and the rows' results do not
// depend on what else the step holds.  The grid is (rows, vectors of all runs / 4).
__global__ __launch_bounds__(256) void rotary_runs_unit_kernel(const void* src, int src_dt, size_t ld_src, TurnRuns runs, const int* positions,
                                                               const float* freq, float mag, float eps) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  int vec = blockIdx.y * 4 + (threadIdx.x >> 6), r = 0;
  while (r < runs.n && vec >= runs.run[r].n_vec) vec -= runs.run[r].n_vec, ++r;
  if (r >= runs.n) return;      // (the whole wave)
  const TurnRun& u = runs.run[r];
  const float p = static_cast<float>(positions[t]);
  const size_t a = static_cast<size_t>(t) * ld_src + u.src_off + static_cast<size_t>(vec) * u.width;
  const size_t b = static_cast<size_t>(t) * u.ld_dst + u.dst_off + static_cast<size_t>(vec) * u.dst_stride;
  float lo[2], hi[2];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int e = 2 * (lane + 64 * j);
    lo[j] = e < u.width ? load_as(src, a + e, src_dt) : 0.f;
    hi[j] = e + 1 < u.width ? load_as(src, a + e + 1, src_dt) : 0.f;
    if (e + 1 < u.dims) {
      const float ang = p * freq[e / 2];
      const float c = cosf(ang) * mag, sn = sinf(ang) * mag;
      const float x = lo[j], y = hi[j];
      lo[j] = x * c - y * sn, hi[j] = y * c + x * sn;
    }
    ss = fmaf(lo[j], lo[j], ss);
    ss = fmaf(hi[j], hi[j], ss);
  }
  float inv = 1.0f;
  if (u.unit) inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(u.width) + eps);
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int e = 2 * (lane + 64 * j);
    if (e < u.width) store_as(u.dst, b + e, u.dst_dt, lo[j] * inv);
    if (e + 1 < u.width) store_as(u.dst, b + e + 1, u.dst_dt, hi[j] * inv);
  }
}

// out[t, h * dv + d] = o[t, h * ldh + d] * sigmoid(g[t, h]) for d < dv: a gate per head on an attention's result, which
// may lie in heads padded to ldh columns.
__global__ __launch_bounds__(256) void head_gate_kernel(const void* o, int o_dt, size_t ldo, int head_stride, const float* g, size_t ldg,
                                                        void* out, int out_dt, size_t ldout, int n_heads, int dv) {
  const size_t t = blockIdx.x;
  for (int e = threadIdx.x; e < n_heads * dv; e += 256) {
    const int h = e / dv, d = e % dv;
    const float v = load_as(o, t * ldo + static_cast<size_t>(h) * head_stride + d, o_dt);
    store_as(out, t * ldout + e, out_dt, v * (1.0f / (1.0f + expf(-g[t * ldg + h]))));
  }
}

// out[t, c] = a[t, c] * table[ids[t], off + c]: rows of a table picked by token, times rows of the step.
__global__ __launch_bounds__(256) void rows_times_table_kernel(const void* a, int a_dt, size_t lda, const void* table, int t_dt, size_t ldt,
                                                               int off, const int* ids, int n_rows, void* out, int out_dt, size_t ldo,
                                                               int n) {
  const size_t t = blockIdx.x;
  const int id = ids[t];
  for (int c = threadIdx.x; c < n; c += 256) {
    // (an id outside the table gives NaN, never a neighbour's row; the host refuses it first)
    const float e = (id >= 0 && id < n_rows) ? load_as(table, static_cast<size_t>(id) * ldt + off + c, t_dt) : __builtin_nanf("");
    store_as(out, t * ldo + c, out_dt, load_as(a, t * lda + c, a_dt) * e);
  }
}

// A token input in one launch, for steps of few rows (where five launches cost more than their work): with e the `dim`
// columns from `off` of the table's row that the row's token picks, g = gelu_tanh(W_gate x) * e, y = W_proj g,
// x += y / sqrt(mean(y^2) + eps) * weight.  One workgroup of sixteen waves a row: the stream's row goes to LDS; a wave
// takes a column of g at a time (the row times a row of W_gate, summed over the wave), g in LDS; then a thread a column of
// y (a row of W_proj times g), y in LDS; the squares summed wave by wave in order.  W_gate [dim, width] and W_proj
// [width, dim] in rows, 32-bit or bfloat16; sums in 32-bit.  VEC: bfloat16 matrices whose rows are whole pieces of 16
// bytes: a lane asks for 16 bytes at a time and for all of a column's pieces before it uses the first.
template <bool VEC>
__global__ __launch_bounds__(1024) void token_input_kernel(float* x, size_t ldx, const void* wg, const void* wp, int w_dt, const void* table,
                                                           int t_dt, size_t ldt, int off, const int* ids, int n_rows, const float* weight,
                                                           int width, int dim, float eps, const float* next_w, float next_eps,
                                                           void* next_out, int next_dt, size_t ldn) {
  extern __shared__ float lds[];      // the row [width], g [dim], y [width]
  __shared__ float sh[16];
  float* xs = lds;
  float* g = lds + width;
  float* y = g + dim;
  float* row = x + static_cast<size_t>(blockIdx.x) * ldx;
  const int id = ids[blockIdx.x];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = threadIdx.x; c < width; c += 1024) xs[c] = row[c];
  __syncthreads();
  // (a wave takes four columns of g at a time, j0 + 16 m, and asks for a piece of each of their rows before it uses the first)
  for (int j0 = wave; j0 < dim; j0 += 64) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (VEC) {
      const uint4* wrow[4];
#pragma unroll
      for (int m = 0; m < 4; ++m)
        wrow[m] = reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(wg) + static_cast<size_t>(min(j0 + 16 * m, dim - 1)) * width);
#pragma unroll 2
      for (int p = lane; p < width / 8; p += 64) {
        uint4 w[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) w[m] = wrow[m][p];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const uint32_t q[4] = {w[m].x, w[m].y, w[m].z, w[m].w};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            acc[m] = fmaf(__uint_as_float(q[k] << 16), xs[8 * p + 2 * k], acc[m]);
            acc[m] = fmaf(__uint_as_float(q[k] & 0xffff0000u), xs[8 * p + 2 * k + 1], acc[m]);
          }
        }
      }
    } else {
      for (int c = lane; c < width; c += 64) {
#pragma unroll
        for (int m = 0; m < 4; ++m)
          acc[m] = fmaf(load_as(wg, static_cast<size_t>(min(j0 + 16 * m, dim - 1)) * width + c, w_dt), xs[c], acc[m]);
      }
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int j = j0 + 16 * m;
      const float v = wave_sum(acc[m]);
      if (lane == 0 && j < dim) {
        const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
        const float e = (id >= 0 && id < n_rows) ? load_as(table, static_cast<size_t>(id) * ldt + off + j, t_dt) : __builtin_nanf("");
        g[j] = 0.5f * v * (1.0f + tanhf(u)) * e;
      }
    }
  }
  __syncthreads();
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += 1024) {
    float acc = 0.f;
    if (VEC) {
      const uint4* wrow = reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(wp) + static_cast<size_t>(c) * dim);
#pragma unroll 8
      for (int p = 0; p < dim / 8; ++p) {
        const uint4 w = wrow[p];
        const uint32_t q[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          acc = fmaf(__uint_as_float(q[k] << 16), g[8 * p + 2 * k], acc);
          acc = fmaf(__uint_as_float(q[k] & 0xffff0000u), g[8 * p + 2 * k + 1], acc);
        }
      }
    } else {
      for (int j = 0; j < dim; ++j) acc = fmaf(load_as(wp, static_cast<size_t>(c) * dim + j, w_dt), g[j], acc);
    }
    y[c] = acc;
    ss = fmaf(acc, acc, ss);
  }
  ss = wave_sum(ss);
  if (lane == 0) sh[wave] = ss;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < 16; ++w) total += sh[w];
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  float after = 0.f;
  for (int c = threadIdx.x; c < width; c += 1024) {
    const float sum = fmaf(y[c] * inv, weight ? weight[c] : 1.0f, xs[c]);
    row[c] = sum;
    y[c] = sum;      // (the thread's own place)
    after = fmaf(sum, sum, after);
  }
  if (!next_out) return;
  // the norm that reads the stream next, on the row as it stands now
  after = wave_sum(after);
  __syncthreads();
  if (lane == 0) sh[wave] = after;
  __syncthreads();
  total = 0.f;
#pragma unroll
  for (int w = 0; w < 16; ++w) total += sh[w];
  const float inv2 = 1.0f / sqrtf(total / static_cast<float>(width) + next_eps);
  for (int c = threadIdx.x; c < width; c += 1024)
    store_as(next_out, static_cast<size_t>(blockIdx.x) * ldn + c, next_dt, next_w ? y[c] * inv2 * next_w[c] : y[c] * inv2);
}

// ---- activations of projections that feed a recurrence or a gate --------------------------------------------
enum { ACT_SILU = 0, ACT_SIGMOID = 1, ACT_TANH = 2, ACT_EXP_NEG_EXP = 3, ACT_BOUNDED_SIGMOID = 4, ACT_EXP_NEG_SOFTPLUS = 5, ACT_XIELU = 6,
       ACT_RELU2 = 7 };

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// log(1 + e^z), without overflow
__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

__device__ __forceinline__ float activation(int kind, float z, float lower) {
  switch (kind) {
    case ACT_EXP_NEG_SOFTPLUS: return expf(-lower * softplus_f(z));      // (lower: the rate of the column)
    case ACT_SILU: return z * sigmoid_f(z);
    case ACT_SIGMOID: return sigmoid_f(z);
    case ACT_TANH: return tanhf(z);
    case ACT_EXP_NEG_EXP: return expf(-expf(z));
    case ACT_RELU2: return fmaxf(z, 0.f) * fmaxf(z, 0.f);
    default: return lower + (1.0f - lower) * sigmoid_f(z);
  }
}

// out[t, c] = act(x[t, c] + bias[c]) (lower[c]: the least value of a bounded sigmoid, or the rate of exp(-rate softplus(z)));
// "xielu" has two numbers for all columns in `lower`, (a, b): z > 0: a z^2 + z / 2; else b (e^z - 1 - z) + z / 2
__global__ __launch_bounds__(256) void activate_kernel(const float* x, size_t ldx, const float* bias, const float* lower, int kind,
                                                       void* out, int out_dt, size_t ldo, int n) {
  const int t = blockIdx.x;
  if (kind == ACT_XIELU) {
    const float a = lower[0], b = lower[1];
    for (int c = threadIdx.x; c < n; c += 256) {
      const float z = x[t * ldx + c] + (bias ? bias[c] : 0.f);
      store_as(out, t * ldo + c, out_dt, z > 0.f ? fmaf(a * z, z, 0.5f * z) : fmaf(b, expm1f(z) - z, 0.5f * z));
    }
    return;
  }
  for (int c = threadIdx.x; c < n; c += 256) {
    const float z = x[t * ldx + c] + (bias ? bias[c] : 0.f);
    store_as(out, t * ldo + c, out_dt, activation(kind, z, lower ? lower[c] : 0.f));
  }
}

// out[t, h, :] = x[t, h, :] / sqrt(sum(x[t, h, :]^2) + eps) * scale: every head's vector made a unit vector; a wave a head
__global__ __launch_bounds__(64) void unit_heads_kernel(const float* x, size_t ldx, float* out, size_t ldo, int dim, float eps, float scale) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* src = x + t * ldx + static_cast<size_t>(h) * dim;
  float ss = 0.f;
  for (int j = lane; j < dim; j += 64) ss = fmaf(src[j], src[j], ss);
  ss = wave_sum(ss);
  const float inv = scale / sqrtf(ss + eps);
  for (int j = lane; j < dim; j += 64) out[t * ldo + static_cast<size_t>(h) * dim + j] = src[j] * inv;
}

// out[t, c] = x[t, c] * act(g[t, c])
__global__ __launch_bounds__(256) void gated_kernel(const void* x, int x_dt, size_t ldx, const float* g, size_t ldg, int kind,
                                                    void* out, int out_dt, size_t ldo, int n) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < n; c += 256)
    store_as(out, t * ldo + c, out_dt, load_as(x, t * ldx + c, x_dt) * activation(kind, g[t * ldg + c], 0.f));
}

// ---- the scan ----------------------------------------------------------------------------------------------
// Per request, head and 16 (or 4) value columns one wave keeps the head's state S [dk][those columns] in registers and
// walks the request's rows of this step in order:
//   a_i = key_from_decay ? 1 - w_i : k_i
//   read_after:   S_i <- w_i S_i + a_i v_j ;  o_j = sum_i r_i S_i
//   delta:        S_i <- w_i S_i ;  e_j = beta (v_j - sum_i a_i S_i) ;  S_i <- S_i + a_i e_j ;  o_j = sum_i r_i S_i
//   else:         o_j = sum_i r_i (S_i + u_i a_i v_j) ;  S_i <- w_i S_i + a_i v_j
// w is a number per row, head and key channel, or (w_rows) one per row and head for all the head's channels, or (w_head) one
// per head for all rows and channels.  r and k may have
// fewer heads than v: head h reads r and k of head h / (H / G).
// A column's key channels are shared out among KG lanes that lie side by side (4 lanes for heads of up to 32 key
// channels, 16 beyond), so a wave has 64 / KG columns and a column's parts are joined inside a row of 16 lanes,
// without LDS; a part's sum over i runs in ascending order, one fused multiply-add a step, and the parts are joined
// in one fixed order, whatever the step holds.
// A row's r, k and w reach the lanes through LDS, some rows at a time (16, or 2 in a step of single rows); the next are asked for before the
// current ones are worked on.  Places beyond a request's last row hold r = 0, a = 0, w = 1, which change nothing, so the
// rows of a fetch are worked on without a branch between them.
enum { SCAN_BEFORE = 0, SCAN_AFTER = 1, SCAN_DELTA = 2 };

struct ScanArgs {
  const float *r, *k, *v, *w, *u, *beta, *w_head;
  size_t ldr, ldk, ldv, ldw, ldb;
  int G;
  float* state;
  size_t slot_stride;
  const int *row_start, *slots;
  int H, dk, dv, read_after, key_from_decay, beta_logits, w_rows;
  float* out;
  size_t ldo;
};

template <int DK, int KG, int MODE, bool VEC, int TB>
__global__ __launch_bounds__(64) void scan_kernel(ScanArgs a) {
  constexpr bool AFTER = MODE == SCAN_AFTER, DELTA = MODE == SCAN_DELTA;
  constexpr int KQ = DK / KG;
  constexpr int CW = 64 / KG;      // value columns of a wave
  constexpr int NL = DK >= 64 ? DK / 64 : 1;
  // TB: rows asked for at a time (a trip to memory is paid once per TB rows, not per row; all TB places are worked on,
  // so steps of single rows take a small TB).  A row's sums are the same for every TB.
  constexpr int N4 = TB * DK / 4, NV = N4 >= 64 ? N4 / 64 : 1;      // VEC: groups of four numbers per array, per lane
  __shared__ __attribute__((aligned(16))) float sh[TB][3 * DK];
  __shared__ __attribute__((aligned(16))) float shv[TB][CW];
  __shared__ __attribute__((aligned(16))) float shu[DK];
  __shared__ float shb[TB];
  const int s = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
  const int hq = h / (a.H / a.G);                     // the head of r and k that this head reads
  const float wh = a.w_head ? a.w_head[h] : 1.0f;     // one decay for the head, where w is none
  const int kg = lane % KG, j0 = blockIdx.x * CW, j = j0 + lane / KG;
  const int slot = a.slots[s];
  if (slot < 0) return;
  const int row0 = a.row_start[s], row1 = a.row_start[s + 1];
  if (row0 >= row1) return;
  const bool live = j < a.dv;
  const int dk = a.dk, dv = a.dv;
  // the state lies [head][value column][key channel]: a lane's channels side by side, a column's lanes too
  float* sp = a.state + static_cast<size_t>(slot) * a.slot_stride + (static_cast<size_t>(h) * dv + j) * dk + kg * KQ;
  float S[KQ];
#pragma unroll
  for (int q = 0; q < KQ; ++q) S[q] = (live && kg * KQ + q < dk) ? sp[q] : 0.f;
  for (int i = lane; i < DK; i += 64) shu[i] = (a.u && i < dk) ? a.u[h * dk + i] : 0.f;
  // what a fetch brings: (not VEC) a lane's own numbers row by row; (VEC: every size a multiple of 4 and every row at a
  // multiple of 16 bytes) 16 bytes a lane and load, eight rows of r, k or w in DK / 32 loads: a row then costs a wave
  // 7 / 8 of a vector load where it cost four, and those loads, not the arithmetic, were what a row waited for
  float nr[VEC ? 1 : TB][NL], nk[VEC ? 1 : TB][NL], nw[VEC ? 1 : TB][NL], nv[VEC ? 1 : TB], nb[VEC ? 1 : TB];
  f32x4 r4[VEC ? NV : 1], k4[VEC ? NV : 1], w4[VEC ? NV : 1], v4;
  auto beta_of = [&](float z) { return a.beta_logits ? 1.0f / (1.0f + expf(-z)) : z; };      // (beta given as it is, or as sigmoid's argument)
  auto fetch = [&](int t0) {
    if constexpr (VEC) {
      const f32x4 zero = {0.f, 0.f, 0.f, 0.f}, one = {1.f, 1.f, 1.f, 1.f};
#pragma unroll
      for (int it = 0; it < NV; ++it) {
        const int idx = it * 64 + lane, bq = idx / (DK / 4), i = (idx % (DK / 4)) * 4, t = t0 + bq;
        const bool ok = idx < N4 && t < row1 && i < dk;
        r4[it] = ok ? *reinterpret_cast<const f32x4*>(a.r + t * a.ldr + hq * dk + i) : zero;
        k4[it] = (ok && !a.key_from_decay) ? *reinterpret_cast<const f32x4*>(a.k + t * a.ldk + hq * dk + i) : zero;
        w4[it] = !ok ? one : a.w_head ? one * wh : a.w_rows ? one * a.w[t * a.ldw + h] : *reinterpret_cast<const f32x4*>(a.w + t * a.ldw + h * dk + i);
      }
      if constexpr (DELTA) nb[0] = (lane < TB && t0 + lane < row1) ? beta_of(a.beta[(t0 + lane) * a.ldb + h]) : 0.f;
      const int bq = lane / (CW / 4), col = j0 + (lane % (CW / 4)) * 4, t = t0 + bq;
      v4 = (lane < TB * CW / 4 && t < row1 && col < dv) ? *reinterpret_cast<const f32x4*>(a.v + t * a.ldv + h * dv + col) : zero;
    } else {
#pragma unroll
      for (int bq = 0; bq < TB; ++bq) {
        const int t = t0 + bq;
        const bool row = t < row1;
#pragma unroll
        for (int q = 0; q < NL; ++q) {
          const int i = lane + 64 * q;
          const bool ok = row && i < dk;
          nr[bq][q] = ok ? a.r[t * a.ldr + hq * dk + i] : 0.f;
          nk[bq][q] = (ok && !a.key_from_decay) ? a.k[t * a.ldk + hq * dk + i] : 0.f;
          nw[bq][q] = !ok ? 1.f : a.w_head ? wh : a.w_rows ? a.w[t * a.ldw + h] : a.w[t * a.ldw + h * dk + i];
        }
        if constexpr (DELTA) nb[bq] = row ? beta_of(a.beta[t * a.ldb + h]) : 0.f;
        nv[bq] = (row && live) ? a.v[t * a.ldv + h * dv + j] : 0.f;
      }
    }
  };
  fetch(row0);
  for (int t0 = row0; t0 < row1; t0 += TB) {
    float vj[TB], bj[TB];
    if constexpr (VEC) {
      if constexpr (DELTA) {
        if (lane < TB) shb[lane] = nb[0];
      }
#pragma unroll
      for (int it = 0; it < NV; ++it) {
        const int idx = it * 64 + lane, bq = idx / (DK / 4), i = (idx % (DK / 4)) * 4;
        if (idx < N4) {
          const f32x4 one = {1.f, 1.f, 1.f, 1.f};
          *reinterpret_cast<f32x4*>(&sh[bq][i]) = r4[it];
          *reinterpret_cast<f32x4*>(&sh[bq][DK + i]) = a.key_from_decay ? one - w4[it] : k4[it];
          *reinterpret_cast<f32x4*>(&sh[bq][2 * DK + i]) = w4[it];
        }
      }
      if (lane < TB * CW / 4) *reinterpret_cast<f32x4*>(&shv[lane / (CW / 4)][(lane % (CW / 4)) * 4]) = v4;
    } else {
#pragma unroll
      for (int bq = 0; bq < TB; ++bq) {
#pragma unroll
        for (int q = 0; q < NL; ++q) {
          const int i = lane + 64 * q;
          if (i < DK) {
            sh[bq][i] = nr[bq][q];
            sh[bq][DK + i] = a.key_from_decay ? 1.0f - nw[bq][q] : nk[bq][q];
            sh[bq][2 * DK + i] = nw[bq][q];
          }
        }
        vj[bq] = nv[bq];
        if constexpr (DELTA) bj[bq] = nb[bq];
      }
    }
    __syncthreads();
    if constexpr (VEC) {
#pragma unroll
      for (int bq = 0; bq < TB; ++bq) {
        vj[bq] = shv[bq][lane / KG];
        if constexpr (DELTA) bj[bq] = shb[bq];
      }
    }
    if (t0 + TB < row1) fetch(t0 + TB);
    // (no branch inside the eight rows: their reads, sums and joins can then overlap)
    float ob[TB];
#pragma unroll
    for (int bq = 0; bq < TB; ++bq) {
      const float* mr = sh[bq] + kg * KQ;
      const float* mk = mr + DK;
      const float* mw = mk + DK;
      const float* mu = shu + kg * KQ;
      float o = 0.f;
      if constexpr (DELTA) {
        // the state fades; what it answers to the key is taken off the value; the rest, times beta, is written
        float ans = 0.f;
#pragma unroll
        for (int q = 0; q < KQ; ++q) {
          S[q] *= mw[q];
          ans = fmaf(mk[q], S[q], ans);
        }
        ans = group_reduce<KG>(ans, SumOp());
        const float e = bj[bq] * (vj[bq] - ans);
#pragma unroll
        for (int q = 0; q < KQ; ++q) {
          S[q] = fmaf(mk[q], e, S[q]);
          o = fmaf(mr[q], S[q], o);
        }
        ob[bq] = group_reduce<KG>(o, SumOp());
        continue;
      }
#pragma unroll
      for (int q = 0; q < KQ; ++q) {
        const float kv = mk[q] * vj[bq];
        if (AFTER) {
          S[q] = fmaf(mw[q], S[q], kv);
          o = fmaf(mr[q], S[q], o);
        } else {
          o = fmaf(mr[q], fmaf(mu[q], kv, S[q]), o);
          S[q] = fmaf(mw[q], S[q], kv);
        }
      }
      ob[bq] = group_reduce<KG>(o, SumOp());
    }
    if (live && kg == 0) {
#pragma unroll
      for (int bq = 0; bq < TB; ++bq)
        if (t0 + bq < row1) a.out[(t0 + bq) * a.ldo + h * dv + j] = ob[bq];
    }
    __syncthreads();
  }
  if (live)
#pragma unroll
    for (int q = 0; q < KQ; ++q)
      if (kg * KQ + q < dk) sp[q] = S[q];
}

// ---- a norm per head, with a gate ----------------------------------------------------------------------------
// y = o[t, h, j] (+ skip[t, h * dv + j] * skip_scale[(h * dv + j) / skip_dim], a second summand with a number per run of
// skip_dim columns); gate_first: y *= act(gate) before the norm, else behind it;
// out[t, h, j] = y / sqrt(mean_j(y^2) + eps) * weight[h * w_stride + j]; a wave a head.
struct HeadNormArgs {
  const float* o; size_t ld;
  const float* weight; int w_stride; float eps;
  const float* gate; size_t ldg; int gate_kind, gate_first;
  const float* skip; size_t lds; const float* skip_scale; int skip_dim;
  void* out; int out_dt; size_t ldo; int dv;
};

__device__ __forceinline__ float head_norm_in(const HeadNormArgs& a, size_t t, int col) {
  float y = a.o[t * a.ld + col];
  if (a.skip) y = fmaf(a.skip[t * a.lds + col], a.skip_scale[col / a.skip_dim], y);
  if (a.gate && a.gate_first) y *= activation(a.gate_kind, a.gate[t * a.ldg + col], 0.f);
  return y;
}

__global__ __launch_bounds__(64) void head_norm_kernel(HeadNormArgs a) {
  const int h = blockIdx.y, lane = threadIdx.x, dv = a.dv;
  const size_t t = blockIdx.x;
  float ss = 0.f;
  for (int j = lane; j < dv; j += 64) {
    const float y = head_norm_in(a, t, h * dv + j);
    ss = fmaf(y, y, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(dv) + a.eps);
  for (int j = lane; j < dv; j += 64) {
    float y = head_norm_in(a, t, h * dv + j) * inv;
    if (a.weight) y *= a.weight[h * a.w_stride + j];
    if (a.gate && !a.gate_first) y *= activation(a.gate_kind, a.gate[t * a.ldg + static_cast<size_t>(h) * dv + j], 0.f);
    store_as(a.out, t * a.ldo + static_cast<size_t>(h) * dv + j, a.out_dt, y);
  }
}

// The same for heads of many columns (all heads normed as one vector): a workgroup a head, the sums as in rmsnorm_kernel.
// Which of the two kernels runs depends on the head's size alone.
__global__ __launch_bounds__(256) void head_norm_wide_kernel(HeadNormArgs a) {
  __shared__ float sh[4];
  const int h = blockIdx.y, dv = a.dv;
  const size_t t = blockIdx.x;
  float ss = 0.f;
  for (int j = threadIdx.x; j < dv; j += 256) {
    const float y = head_norm_in(a, t, h * dv + j);
    ss = fmaf(y, y, ss);
  }
  ss = block_sum_256(ss, sh);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(dv) + a.eps);
  for (int j = threadIdx.x; j < dv; j += 256) {
    float y = head_norm_in(a, t, h * dv + j) * inv;
    if (a.weight) y *= a.weight[h * a.w_stride + j];
    if (a.gate && !a.gate_first) y *= activation(a.gate_kind, a.gate[t * a.ldg + static_cast<size_t>(h) * dv + j], 0.f);
    store_as(a.out, t * a.ldo + static_cast<size_t>(h) * dv + j, a.out_dt, y);
  }
}

// head_norm_wide_kernel for heads of up to 256 NC columns: a thread's share of the head stays in registers between the sum and
// the stores (one trip to memory where the kernel above makes two).  The same sums in the same order: the same bits.
template <int NC>
__global__ __launch_bounds__(256) void head_norm_held_kernel(HeadNormArgs a) {
  __shared__ float sh[4];
  const int h = blockIdx.y, dv = a.dv;
  const size_t t = blockIdx.x;
  float y[NC], w[NC], gt[NC];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NC; ++k) {
    const int j = threadIdx.x + 256 * k;
    const bool ok = j < dv;
    const int jj = ok ? j : 0;
    y[k] = ok ? head_norm_in(a, t, h * dv + jj) : 0.f;
    w[k] = a.weight ? a.weight[h * a.w_stride + jj] : 1.0f;
    gt[k] = (a.gate && !a.gate_first) ? a.gate[t * a.ldg + static_cast<size_t>(h) * dv + jj] : 0.f;
  }
#pragma unroll
  for (int k = 0; k < NC; ++k)
    if (threadIdx.x + 256 * k < dv) ss = fmaf(y[k], y[k], ss);
  ss = block_sum_256(ss, sh);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(dv) + a.eps);
#pragma unroll
  for (int k = 0; k < NC; ++k) {
    const int j = threadIdx.x + 256 * k;
    if (j < dv) {
      float v = y[k] * inv;
      if (a.weight) v *= w[k];
      if (a.gate && !a.gate_first) v *= activation(a.gate_kind, gt[k], 0.f);
      store_as(a.out, t * a.ldo + static_cast<size_t>(h) * dv + j, a.out_dt, v);
    }
  }
}

// ---- what a state-space recurrence with one decay per head reads -------------------------------------------------
// dt = log(1 + e^(z[t, h] + bias[h])); decay[t, h] = exp(-rate[h] * dt); v[t, h, :] = dt * x[t, h, :].  A workgroup a row.
__global__ __launch_bounds__(256) void step_sizes_kernel(const float* z, size_t ldz, const float* bias, const float* rate, const float* x,
                                                         size_t ldx, int H, int dv, float* decay, size_t ldd, float* v, size_t ldv) {
  const size_t t = blockIdx.x;
  for (int h = threadIdx.x; h < H; h += 256) decay[t * ldd + h] = expf(-rate[h] * softplus_f(z[t * ldz + h] + (bias ? bias[h] : 0.f)));
  for (int c = threadIdx.x; c < H * dv; c += 256) {
    const int h = c / dv;
    v[t * ldv + c] = softplus_f(z[t * ldz + h] + (bias ? bias[h] : 0.f)) * x[t * ldx + c];
  }
}

// ---- a recurrence of single numbers whose gates read the token alone ----------------------------------------------
// z = sigmoid(a[t, c] + bias_a[c]); u = b[t, c] + bias_b[c]; cand = u >= 0 ? u + 1/2 : sigmoid(u); S <- (1 - z) S + z cand;
// out[t, c] = S * silu(g[t, c]).  A workgroup owns 64 channels of a request, a lane a channel.  Its WAVES waves take
// eight rows each of every run of 8 WAVES rows: a wave first walks its rows from a state of zero, which gives the
// product P of its (1 - z) and what it adds, Q, so that the state behind its rows is P S + Q for any state S before
// them; the waves' (P, Q) meet in LDS, every wave folds those of the waves before it into the state at the run's
// start, in order, and walks its rows again from there.  A step of single rows takes one wave, which walks them once.
// A row's result depends on the rows before it alone; how the rows were cut changes it by rounding only.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gate_scan_kernel(const float* a, size_t lda, const float* b, size_t ldb, const float* g,
                                                               size_t ldg, const float* bias_a, const float* bias_b, float* state,
                                                               size_t slot_stride, const int* row_start, const int* slots, int width,
                                                               void* out, int out_dt, size_t ldo) {
  constexpr int TB = 8;
  __shared__ float shp[2][WAVES][64], shq[2][WAVES][64];
  const int s = blockIdx.y, lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int c = blockIdx.x * 64 + lane;
  const int slot = slots[s];
  if (slot < 0) return;      // (the whole workgroup)
  const int row0 = row_start[s], row1 = row_start[s + 1];
  if (row0 >= row1) return;
  const bool live = c < width;
  const int cc = live ? c : width - 1;
  const float ba = bias_a ? bias_a[cc] : 0.f, bb = bias_b ? bias_b[cc] : 0.f;
  float* sp = state + static_cast<size_t>(slot) * slot_stride + cc;
  float S0 = *sp;      // the state before the run that is worked on; every wave keeps it
  float na[TB], nb[TB], ng[TB];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const size_t t = min(t0 + i, row1 - 1);
      na[i] = a[t * lda + cc], nb[i] = b[t * ldb + cc], ng[i] = g[t * ldg + cc];
    }
  };
  fetch(row0 + wave * TB);
  int par = 0;
  for (int t0 = row0; t0 < row1; t0 += WAVES * TB, par ^= 1) {
    const int mine = t0 + wave * TB;
    float keep[TB], add[TB], gate[TB];
    float P = 1.f, Q = 0.f;
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const float z = sigmoid_f(na[i] + ba), u = nb[i] + bb;
      const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
      const bool row = mine + i < row1;
      keep[i] = row ? 1.0f - z : 1.0f;      // (places beyond the last row change nothing)
      add[i] = row ? z * cand : 0.f;
      gate[i] = ng[i];
      P *= keep[i];
      Q = fmaf(keep[i], Q, add[i]);
    }
    if (t0 + WAVES * TB < row1) fetch(mine + WAVES * TB);
    float S = S0;
    if constexpr (WAVES > 1) {
      shp[par][wave][lane] = P, shq[par][wave][lane] = Q;
      __syncthreads();      // (the other half of LDS is what the run before used: one barrier a run)
      float run = S0;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        if (w == wave) S = run;
        run = fmaf(shp[par][w][lane], run, shq[par][w][lane]);
      }
      S0 = run;
    }
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      S = fmaf(keep[i], S, add[i]);
      if (live && mine + i < row1)
        store_as(out, static_cast<size_t>(mine + i) * ldo + c, out_dt, S * activation(ACT_SILU, gate[i], 0.f));
    }
    if constexpr (WAVES == 1) S0 = S;
  }
  if (live && wave == 0) *sp = S0;
}

// ---- a state per channel and state index with a decay of its own (the selective scan) -----------------------------
// Over each request's rows in order, per channel c and state index n:
//   dt = log(1 + e^(dt_in[t, c] + dt_bias[c]));  S[c, n] <- exp(dt A[c, n]) S[c, n] + dt x[t, c] B[t, n]
//   y[t, c] = sum_n S[c, n] C[t, n] + D[c] x[t, c];  out[t, c] = y * silu(z[t, c])
// x is what a short convolution and its activation left, 32-bit or bfloat16; everything else that enters is 32-bit.
// A channel lies on 16 neighbouring lanes; lane l of them keeps the states n = l, l + 16, ... (PER of them) in registers
// from a portion's first row to its last, and the sum over n is joined inside the row of 16 lanes, always in one order.
// The rows are asked for TB at a time.  The same kernel for portions and for decoded tokens; a row's result depends on
// the state before it alone, so how a prompt is cut changes nothing.
struct SelectiveArgs {
  const void* x;      // 32-bit or bfloat16 (x_dt): what the convolution left
  int x_dt;
  const float *dt, *dt_bias, *B, *C, *A, *D, *z;
  size_t ldx, ldd, ldb, ldc, ldz;
  float* state;
  size_t slot_stride;
  const int *row_start, *slots;
  int inner, N;
  void* out;
  int out_dt;
  size_t ldo;
};

// CG: a lane works on that many channels (16 CG channels a workgroup), each with its own loads in flight: a step of
// single rows, whose work is one trip to memory and back per channel, then needs a quarter of the waves.
template <int PER, int CG, int TB>
__global__ __launch_bounds__(256) void selective_scan_kernel(SelectiveArgs a) {
  const int s = blockIdx.y;
  const int slot = a.slots[s];
  if (slot < 0) return;      // (the whole workgroup: padding of a captured step)
  const int row0 = a.row_start[s], row1 = a.row_start[s + 1];
  if (row0 >= row1) return;
  const int l = threadIdx.x & 15;
  float rate[CG][PER], S[CG][PER], bias[CG], skip[CG];
  int nn[PER], cc[CG];
  bool live[CG];
  float* sp[CG];
#pragma unroll
  for (int j = 0; j < PER; ++j) nn[j] = l + 16 * j < a.N ? l + 16 * j : 0;
#pragma unroll
  for (int g = 0; g < CG; ++g) {
    const int c = (blockIdx.x * CG + g) * 16 + (threadIdx.x >> 4);
    live[g] = c < a.inner;
    cc[g] = live[g] ? c : a.inner - 1;
    sp[g] = a.state + static_cast<size_t>(slot) * a.slot_stride + static_cast<size_t>(cc[g]) * a.N;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const bool has = l + 16 * j < a.N;
      rate[g][j] = has ? a.A[static_cast<size_t>(cc[g]) * a.N + nn[j]] : 0.f;      // (a place beyond N: decay 1 on a state of 0, B and C read as 0)
      S[g][j] = has ? sp[g][nn[j]] : 0.f;
    }
    bias[g] = a.dt_bias ? a.dt_bias[cc[g]] : 0.f, skip[g] = a.D ? a.D[cc[g]] : 0.f;
  }
  float fx[CG][TB], fd[CG][TB], fz[CG][TB], fb[TB][PER], fc[TB][PER];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const size_t t = min(t0 + i, row1 - 1);
#pragma unroll
      for (int g = 0; g < CG; ++g) {
        fx[g][i] = load_as(a.x, t * a.ldx + cc[g], a.x_dt), fd[g][i] = a.dt[t * a.ldd + cc[g]];
        fz[g][i] = a.z ? a.z[t * a.ldz + cc[g]] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < PER; ++j) fb[i][j] = a.B[t * a.ldb + nn[j]], fc[i][j] = a.C[t * a.ldc + nn[j]];
    }
  };
  fetch(row0);
  for (int t0 = row0; t0 < row1; t0 += TB) {
    float x[CG][TB], d[CG][TB], z[CG][TB], b[TB][PER], cm[TB][PER];
#pragma unroll
    for (int i = 0; i < TB; ++i) {
#pragma unroll
      for (int g = 0; g < CG; ++g) x[g][i] = fx[g][i], d[g][i] = fd[g][i], z[g][i] = fz[g][i];
#pragma unroll
      for (int j = 0; j < PER; ++j) b[i][j] = fb[i][j], cm[i][j] = fc[i][j];
    }
    if (t0 + TB < row1) fetch(t0 + TB);
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      if (t0 + i >= row1) break;
#pragma unroll
      for (int g = 0; g < CG; ++g) {
        const float dt = softplus_f(d[g][i] + bias[g]);
        const float dx = dt * x[g][i];
        float y = 0.f;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
          const bool has = l + 16 * j < a.N;
          S[g][j] = fmaf(expf(dt * rate[g][j]), S[g][j], has ? dx * b[i][j] : 0.f);
          y = fmaf(S[g][j], has ? cm[i][j] : 0.f, y);
        }
        y = group_reduce<16>(y, SumOp());
        if (live[g] && l == 0) {
          y = fmaf(skip[g], x[g][i], y);
          if (a.z) y *= z[g][i] / (1.0f + expf(-z[g][i]));
          store_as(a.out, static_cast<size_t>(t0 + i) * a.ldo + cc[g], a.out_dt, y);
        }
      }
    }
  }
#pragma unroll
  for (int g = 0; g < CG; ++g) {
    if (!live[g]) continue;
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (l + 16 * j < a.N) sp[g][l + 16 * j] = S[g][j];
  }
}

// lane i's value of each row of 16 lanes, in all lanes of the row (i is a constant once the caller's loop is unrolled)
__device__ __forceinline__ float row_share(float v, int i) {
  switch (i & 15) {
    case 0: return dpp_move<0x150>(v);
    case 1: return dpp_move<0x151>(v);
    case 2: return dpp_move<0x152>(v);
    case 3: return dpp_move<0x153>(v);
    case 4: return dpp_move<0x154>(v);
    case 5: return dpp_move<0x155>(v);
    case 6: return dpp_move<0x156>(v);
    case 7: return dpp_move<0x157>(v);
    case 8: return dpp_move<0x158>(v);
    case 9: return dpp_move<0x159>(v);
    case 10: return dpp_move<0x15A>(v);
    case 11: return dpp_move<0x15B>(v);
    case 12: return dpp_move<0x15C>(v);
    case 13: return dpp_move<0x15D>(v);
    case 14: return dpp_move<0x15E>(v);
    default: return dpp_move<0x15F>(v);
  }
}

// The same recurrence for long portions of few requests, where a wave that walks a request's rows alone leaves the chip
// idle: a workgroup's WAVES waves take TB rows each (TB <= 8) of every run of WAVES * TB rows.  A wave first walks its
// rows from a state of zero, which gives, per state, the product P of its decays and what it adds, Q, so that the state
// behind its rows is P S + Q for any state S before them; the waves' (P, Q) meet in LDS, every wave folds those of the
// waves before it into the state at the run's start, in order, and walks its rows again from there (the decays and
// summands are kept from the first walk).  What is one number per row and channel is made once, not by all 16 lanes of
// the channel: lane i of them (i < TB) has row i's step (softplus) and step * x, lane 8 + i its silu(z) and x, and the
// others read them from there (DPP row_share).  The decays are 2^(step * A log2(e)) by the hardware's exponential.
// A row's result depends on the rows before it alone; how the rows were cut changes it by rounding only, where the
// kernel above gives the same bits.
template <int PER, int WAVES, int TB>
__global__ __launch_bounds__(WAVES * 64) void selective_scan_runs_kernel(SelectiveArgs a) {
  static_assert(TB <= 8, "a row's step lies on lane i, its gate on lane 8 + i of the channel's 16");
  __shared__ float shp[2][WAVES][PER][64], shq[2][WAVES][PER][64];
  const int s = blockIdx.y;
  const int slot = a.slots[s];
  if (slot < 0) return;      // (the whole workgroup)
  const int row0 = a.row_start[s], row1 = a.row_start[s + 1];
  if (row0 >= row1) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l = lane & 15;
  const int c = blockIdx.x * 4 + (lane >> 4);
  const bool live = c < a.inner;
  const int cc = live ? c : a.inner - 1;
  float rate[PER], S0[PER];
  int nn[PER];
  float* sp = a.state + static_cast<size_t>(slot) * a.slot_stride + static_cast<size_t>(cc) * a.N;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = l + 16 * j;
    const bool has = n < a.N;
    nn[j] = has ? n : 0;
    rate[j] = has ? a.A[static_cast<size_t>(cc) * a.N + n] * 1.4426950408889634f : 0.f;
    S0[j] = has ? sp[n] : 0.f;      // the state before the run that is worked on; every wave keeps it
  }
  const float bias = a.dt_bias ? a.dt_bias[cc] : 0.f, skip = a.D ? a.D[cc] : 0.f;
  const bool steps = l < 8;              // this lane makes a row's step; else its gate
  const int my = l & 7;                  // the row of the wave's TB that this lane makes them for
  float fx, fs, fb[TB][PER], fc[TB][PER];
  auto fetch = [&](int t0) {
    const size_t t = min(t0 + min(my, TB - 1), row1 - 1);
    fx = load_as(a.x, t * a.ldx + cc, a.x_dt);
    fs = steps ? a.dt[t * a.ldd + cc] : (a.z ? a.z[t * a.ldz + cc] : 0.f);
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const size_t r = min(t0 + i, row1 - 1);
#pragma unroll
      for (int j = 0; j < PER; ++j) fb[i][j] = a.B[r * a.ldb + nn[j]], fc[i][j] = a.C[r * a.ldc + nn[j]];
    }
  };
  fetch(row0 + wave * TB);
  int par = 0;
  for (int t0 = row0; t0 < row1; t0 += WAVES * TB, par ^= 1) {
    const int mine = t0 + wave * TB;
    // lanes 0 .. 7: (step, step * x) of row `my`; lanes 8 .. 15: (silu(z) or 1, D x) of row `my`
    float first, second;
    if (steps) {
      first = softplus_f(fs + bias);
      second = first * fx;
    } else {
      first = a.z ? fs / (1.0f + expf(-fs)) : 1.0f;
      second = skip * fx;
    }
    float keep[TB][PER], add[TB][PER], cm[TB][PER];
    float P[PER], Q[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) P[j] = 1.f, Q[j] = 0.f;
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const bool row = mine + i < row1;
      const float dt = row_share(first, i), dx = row_share(second, i);
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        const bool has = l + 16 * j < a.N;
        keep[i][j] = row ? __builtin_amdgcn_exp2f(dt * rate[j]) : 1.0f;      // (places beyond the last row change nothing)
        add[i][j] = (row && has) ? dx * fb[i][j] : 0.f;
        cm[i][j] = has ? fc[i][j] : 0.f;
        P[j] *= keep[i][j];
        Q[j] = fmaf(keep[i][j], Q[j], add[i][j]);
      }
    }
    if (t0 + WAVES * TB < row1) fetch(mine + WAVES * TB);
    float S[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) shp[par][wave][j][lane] = P[j], shq[par][wave][j][lane] = Q[j];
    __syncthreads();      // (the other half of LDS is what the run before used: one barrier a run)
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      float run = S0[j];
      S[j] = run;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        if (w == wave) S[j] = run;
        run = fmaf(shp[par][w][j][lane], run, shq[par][w][j][lane]);
      }
      S0[j] = run;
    }
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      float y = 0.f;
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        S[j] = fmaf(keep[i][j], S[j], add[i][j]);
        y = fmaf(S[j], cm[i][j], y);
      }
      y = group_reduce<16>(y, SumOp());
      const float gate = row_share(first, 8 + i), dx = row_share(second, 8 + i);
      if (live && l == 0 && mine + i < row1) store_as(a.out, static_cast<size_t>(mine + i) * a.ldo + c, a.out_dt, (y + dx) * gate);
    }
  }
  if (live && wave == 0) {
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (l + 16 * j < a.N) sp[l + 16 * j] = S0[j];
  }
}

// ---- queries and keys normed as whole vectors, keys and values to the cache -----------------------------------------
// A row of z is [q: qw | k: kw].  q_out[t] = q / rms(q) * wq; the key that goes to the cache is k / rms(k) * wk, the value
// k as it is (pools [page][key head][offset][dim] and [page][key head][dim][offset], the row's place from slot_map; a
// negative place: nothing is written).  One workgroup a row, the sums as in rmsnorm_kernel.
__global__ __launch_bounds__(256) void norm_pair_write_kernel(const float* z, size_t ldz, int qw, int kw, const float* wq, const float* wk,
                                                              float eps, void* q_out, size_t ldq, const int* slot_map, void* k_pool,
                                                              void* v_pool, int dh, int page_size, int dt, int write) {
  __shared__ float sh[4];
  const size_t t = blockIdx.x;
  const float* row = z + t * ldz;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < qw; c += 256) sq = fmaf(row[c], row[c], sq);
  for (int c = threadIdx.x; c < kw; c += 256) sk = fmaf(row[qw + c], row[qw + c], sk);
  sq = block_sum_256(sq, sh);
  sk = block_sum_256(sk, sh);
  const float iq = 1.0f / sqrtf(sq / static_cast<float>(qw) + eps), ik = 1.0f / sqrtf(sk / static_cast<float>(kw) + eps);
  for (int c = threadIdx.x; c < qw; c += 256) store_as(q_out, t * ldq + c, dt, row[c] * iq * wq[c]);
  const int slot = slot_map[t];
  if (!write || slot < 0) return;
  const int page = slot / page_size, off = slot % page_size, Hkv = kw / dh;
  for (int c = threadIdx.x; c < kw; c += 256) {
    const int h = c / dh, d = c % dh;
    const size_t base = (static_cast<size_t>(page) * Hkv + h) * page_size * dh;
    const float k = row[qw + c];
    store_as(k_pool, base + static_cast<size_t>(off) * dh + d, dt, k * ik * wk[c]);
    store_as(v_pool, base + static_cast<size_t>(d) * page_size + off, dt, k);
  }
}

// ---- several copies of the stream -----------------------------------------------------------------------------------
// The stream as n copies [n][rows][width], `plane` numbers apart.
// read: u = sum_s w_in[s] x_s[row] (s ascending, one fused multiply-add a step; w_in none: the plain sum), then
// out[r] = u / sqrt(mean(u^2) + eps) * g (g: a number per column; none, with eps < 0: u itself).  One workgroup a row.
constexpr int STREAMS_MAX = 8;

__global__ __launch_bounds__(256) void streams_read_kernel(const float* xs, size_t plane, int n, const float* w_in, const float* g, float eps,
                                                           void* out, int out_dt, size_t ldo, const int* rows, int width) {
  __shared__ float sh[4];
  const int r = blockIdx.x;
  const size_t src = static_cast<size_t>(rows ? rows[r] : r) * width;
  float wi[STREAMS_MAX];
#pragma unroll
  for (int s = 0; s < STREAMS_MAX; ++s) wi[s] = s < n ? (w_in ? w_in[s] : 1.0f) : 0.f;
  const bool normed = eps >= 0.f;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < n) u = fmaf(wi[s], xs[s * plane + src + c], u);
    ss = fmaf(u, u, ss);
  }
  float inv = 1.0f;
  if (normed) {
    ss = block_sum_256(ss, sh);
    inv = 1.0f / sqrtf(ss / static_cast<float>(width) + eps);
  }
  for (int c = threadIdx.x; c < width; c += 256) {
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < n) u = fmaf(wi[s], xs[s * plane + src + c], u);
    u *= inv;
    store_as(out, static_cast<size_t>(r) * ldo + c, out_dt, g ? u * g[c] : u);
  }
}

// write: every copy anew from the old ones and a sublayer's result y: x_t <- sum_s mix[s][t] x_s + w_out[t] * y (s ascending).
// next_in given: the same workgroup then reads the new copies for the next sublayer, as streams_read_kernel does, into `out`.
// y2 given: the result is the mean of two branches, each normed over the width first with a weight of its own:
// y = (y / rms(y) * by + y2 / rms(y2) * by2) / 2 (the sums as rmsnorm_add_kernel makes them, one branch after the other).
__global__ __launch_bounds__(256) void streams_write_kernel(float* xs, size_t plane, int n, const float* mix, const float* w_out, const float* y,
                                                            size_t ldy, const float* y2, size_t ldy2, const float* by, const float* by2,
                                                            float beps, const float* next_in, const float* g, float eps, void* out,
                                                            int out_dt, size_t ldo, int width) {
  __shared__ float sh[4];
  __shared__ float sm[STREAMS_MAX * STREAMS_MAX + 2 * STREAMS_MAX];
  const size_t row = blockIdx.x;
  if (threadIdx.x < n * n) sm[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < n) {
    sm[STREAMS_MAX * STREAMS_MAX + threadIdx.x] = w_out[threadIdx.x];
    sm[STREAMS_MAX * STREAMS_MAX + STREAMS_MAX + threadIdx.x] = next_in ? next_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const float* wo = sm + STREAMS_MAX * STREAMS_MAX;
  const float* wn = wo + STREAMS_MAX;
  float inv1 = 0.f, inv2 = 0.f;
  if (y2) {
    float s1 = 0.f, s2 = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) {
      const float a = y[row * ldy + c], b = y2[row * ldy2 + c];
      s1 = fmaf(a, a, s1), s2 = fmaf(b, b, s2);
    }
    s1 = block_sum_256(s1, sh);
    s2 = block_sum_256(s2, sh);
    inv1 = 1.0f / sqrtf(s1 / static_cast<float>(width) + beps), inv2 = 1.0f / sqrtf(s2 / static_cast<float>(width) + beps);
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    float old[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s) old[s] = s < n ? xs[s * plane + row * width + c] : 0.f;
    float yc = y[row * ldy + c];
    if (y2) yc = fmaf(0.5f, y2[row * ldy2 + c] * inv2 * by2[c], fmaf(0.5f, yc * inv1 * by[c], 0.f));
    float u = 0.f;
#pragma unroll
    for (int t = 0; t < STREAMS_MAX; ++t) {
      if (t < n) {
        float acc = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s)
          if (s < n) acc = fmaf(sm[s * n + t], old[s], acc);
        acc = fmaf(wo[t], yc, acc);
        xs[t * plane + row * width + c] = acc;
        u = fmaf(wn[t], acc, u);
      }
    }
    ss = fmaf(u, u, ss);
  }
  if (!next_in) return;
  ss = block_sum_256(ss, sh);      // (the barrier inside also orders this workgroup's writes before its reads below)
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(width) + eps);
  for (int c = threadIdx.x; c < width; c += 256) {
    float u = 0.f;
    for (int t = 0; t < n; ++t) u = fmaf(wn[t], xs[t * plane + row * width + c], u);
    u *= inv;
    store_as(out, row * ldo + c, out_dt, g ? u * g[c] : u);
  }
}

// streams_write_kernel for rows of up to 256 NC columns and up to NS copies: a thread's share of the row (the copies, the
// result, the branches' weights) is asked for at once and stays in registers from the first sum to the last store, where the
// kernel above goes to memory three times one behind the other: a decode step's rows wait for those trips, not for bytes.
// The same sums in the same order: the same bits.
template <int NS, int NC>
__global__ __launch_bounds__(256) void streams_write_held_kernel(float* xs, size_t plane, int n, const float* mix, const float* w_out,
                                                                 const float* y, size_t ldy, const float* y2, size_t ldy2, const float* by,
                                                                 const float* by2, float beps, const float* next_in, const float* g,
                                                                 float eps, void* out, int out_dt, size_t ldo, int width) {
  __shared__ float sh[4];
  __shared__ float sm[STREAMS_MAX * STREAMS_MAX + 2 * STREAMS_MAX];
  const size_t row = blockIdx.x;
  float old[NS][NC], yv[NC], y2v[NC], b1[NC], b2[NC], gv[NC];
#pragma unroll
  for (int k = 0; k < NC; ++k) {
    const int c = threadIdx.x + 256 * k;
    const bool ok = c < width;
    const int cc = ok ? c : 0;
    yv[k] = ok ? y[row * ldy + cc] : 0.f;
    y2v[k] = (y2 && ok) ? y2[row * ldy2 + cc] : 0.f;
    b1[k] = y2 ? by[cc] : 0.f, b2[k] = y2 ? by2[cc] : 0.f;
    gv[k] = (next_in && g) ? g[cc] : 1.0f;
#pragma unroll
    for (int s = 0; s < NS; ++s) old[s][k] = (s < n && ok) ? xs[s * plane + row * width + cc] : 0.f;
  }
  if (threadIdx.x < n * n) sm[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < n) {
    sm[STREAMS_MAX * STREAMS_MAX + threadIdx.x] = w_out[threadIdx.x];
    sm[STREAMS_MAX * STREAMS_MAX + STREAMS_MAX + threadIdx.x] = next_in ? next_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const float* wo = sm + STREAMS_MAX * STREAMS_MAX;
  const float* wn = wo + STREAMS_MAX;
  if (y2) {
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int k = 0; k < NC; ++k) s1 = fmaf(yv[k], yv[k], s1), s2 = fmaf(y2v[k], y2v[k], s2);
    s1 = block_sum_256(s1, sh);
    s2 = block_sum_256(s2, sh);
    const float inv1 = 1.0f / sqrtf(s1 / static_cast<float>(width) + beps), inv2 = 1.0f / sqrtf(s2 / static_cast<float>(width) + beps);
#pragma unroll
    for (int k = 0; k < NC; ++k) yv[k] = fmaf(0.5f, y2v[k] * inv2 * b2[k], fmaf(0.5f, yv[k] * inv1 * b1[k], 0.f));
  }
  float ss = 0.f, u[NC];
#pragma unroll
  for (int k = 0; k < NC; ++k) {
    const int c = threadIdx.x + 256 * k;
    u[k] = 0.f;
    if (c < width) {
#pragma unroll
      for (int t = 0; t < NS; ++t) {
        if (t < n) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < NS; ++s)
            if (s < n) acc = fmaf(sm[s * n + t], old[s][k], acc);
          acc = fmaf(wo[t], yv[k], acc);
          xs[t * plane + row * width + c] = acc;
          u[k] = fmaf(wn[t], acc, u[k]);
        }
      }
      ss = fmaf(u[k], u[k], ss);
    }
  }
  if (!next_in) return;
  ss = block_sum_256(ss, sh);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(width) + eps);
#pragma unroll
  for (int k = 0; k < NC; ++k) {
    const int c = threadIdx.x + 256 * k;
    if (c < width) {
      const float v = u[k] * inv;
      store_as(out, row * ldo + c, out_dt, g ? v * gv[k] : v);
    }
  }
}

bool float_kind(int dt) { return dt == DN_F32 || dt == DN_BF16; }

}  // namespace

extern "C" {

int dn_rmsnorm(const void* x, int x_dt, long long ldx, const float* weight, void* out, int out_dt, long long ldo, const int* rows,
               int R, int width, float eps, hipStream_t stream) {
  if (!float_kind(x_dt) || !float_kind(out_dt)) return DN_ERR_DTYPE;
  if (R < 0 || width < 1) return DN_ERR_SHAPE;
  if (R == 0) return 0;
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(R), dim3(256), 0, stream, x, x_dt, static_cast<size_t>(ldx), weight, out, out_dt,
                     static_cast<size_t>(ldo), rows, width, eps);
  return dn_launch_status();
}

int dn_rmsnorm_add(const void* y, int y_dt, long long ldy, const float* weight, const float* scale, float mult, float* x, long long ldx,
                   int T, int width, float eps, const float* gate, long long ldg, const float* next_w, float next_eps, void* next_out,
                   int next_dt, long long ldn, hipStream_t stream) {
  if (!float_kind(y_dt) || (next_out && !float_kind(next_dt))) return DN_ERR_DTYPE;
  if (T < 0 || width < 1 || (gate && ldg < width) || (next_out && ldn < width)) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(rmsnorm_add_kernel, dim3(T), dim3(256), 0, stream, y, y_dt, static_cast<size_t>(ldy), weight, scale, mult, x,
                     static_cast<size_t>(ldx), width, eps, gate, static_cast<size_t>(ldg), next_w, next_eps, next_out, next_dt,
                     static_cast<size_t>(ldn));
  return dn_launch_status();
}

int dn_depth_mix(const float* hist, long long plane, int n, const float* w, float* out, long long total, hipStream_t stream) {
  if (n < 1 || plane < total) return DN_ERR_SHAPE;
  const int vec = plane % 4 == 0 && reinterpret_cast<uintptr_t>(hist) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  if (total == 0) return 0;
  const long long groups = (total + 3) / 4;
  hipLaunchKernelGGL(depth_mix_kernel, dim3(static_cast<unsigned>((groups + 255) / 256)), dim3(256), 0, stream, hist,
                     static_cast<size_t>(plane), n, w, out, static_cast<size_t>(total), vec);
  return dn_launch_status();
}

int dn_unit_heads(const float* x, long long ldx, float* out, long long ldo, int T, int H, int dim, float eps, float scale,
                  hipStream_t stream) {
  if (H < 1 || dim < 1) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(unit_heads_kernel, dim3(T, H), dim3(64), 0, stream, x, static_cast<size_t>(ldx), out, static_cast<size_t>(ldo), dim,
                     eps, scale);
  return dn_launch_status();
}

int dn_concat_cast(const float* a, long long lda, int wa, const float* b, long long ldb, int wb, void* out, int out_dt, int T,
                   hipStream_t stream) {
  if (!float_kind(out_dt)) return DN_ERR_DTYPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(concat_kernel, dim3(T), dim3(256), 0, stream, a, static_cast<size_t>(lda), wa, b, static_cast<size_t>(ldb), wb,
                     out, out_dt);
  return dn_launch_status();
}

int dn_conv_rows(const float* h, long long ldh, const float* w, const float* bias, const float* hist, const int* row_start, const int* slots, int S, int T,
                 int width, int taps, int identity, int silu, void* out, int out_dt, long long ldo, long long hist_stride,
                 hipStream_t stream) {
  if (!float_kind(out_dt)) return DN_ERR_DTYPE;
  if (taps < 1 || S < 1 || ldh < width || ldo < width) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  // (few rows: a workgroup for every 256 channels of a row, so that a step of decoded tokens is more than a handful of workgroups)
  hipLaunchKernelGGL(conv_rows_kernel, dim3(T, T <= 256 ? (width + 255) / 256 : 1), dim3(256), 0, stream, h, static_cast<size_t>(ldh), w, bias, hist, row_start, slots, S, width,
                     taps, identity, silu, out, out_dt, static_cast<size_t>(ldo), static_cast<size_t>(hist_stride));
  return dn_launch_status();
}

int dn_conv_heads(const float* h, long long ldh, const float* w, const float* hist, const int* row_start, const int* slots, int S, int T,
                  int taps, int n_unit, int unit_dim, int n_a, float scale_a, float scale_b, float eps, int n_rest, int rest_dim,
                  float* out, long long ldo, long long hist_stride, hipStream_t stream) {
  const long long width = static_cast<long long>(n_unit) * unit_dim + static_cast<long long>(n_rest) * rest_dim;
  if (taps < 1 || S < 1 || n_unit < 0 || n_rest < 0 || n_unit + n_rest < 1 || ldh < width || ldo < width || n_a < 0 || n_a > n_unit)
    return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(conv_heads_kernel, dim3(T, n_unit + n_rest), dim3(64), 0, stream, h, static_cast<size_t>(ldh), w, hist, row_start,
                     slots, S, static_cast<int>(width), taps, n_unit, unit_dim, n_a, scale_a, scale_b, eps, rest_dim, out,
                     static_cast<size_t>(ldo), static_cast<size_t>(hist_stride));
  return dn_launch_status();
}

// runs: n x 9 numbers (dst, dst_dt, ld_dst, src_off, dst_off, dst_stride, n_vec, width, dims), n <= 3
int dn_rotary_runs(const void* src, int src_dt, long long ld_src, const long long* runs, int n, const int* positions, const float* freq,
                   int T, float mag, long long unit_mask, float eps, hipStream_t stream) {
  if (!float_kind(src_dt) || n < 1 || n > 3) return n < 1 || n > 3 ? DN_ERR_SHAPE : DN_ERR_DTYPE;
  TurnRuns r{};
  r.n = n;
  long long vectors = 0;
  for (int i = 0; i < n; ++i) {
    const long long* q = runs + 9 * i;
    r.run[i] = TurnRun{reinterpret_cast<void*>(q[0]), static_cast<int>(q[1]), static_cast<size_t>(q[2]), static_cast<int>(q[3]),
                       static_cast<int>(q[4]), static_cast<int>(q[5]), static_cast<int>(q[6]), static_cast<int>(q[7]),
                       static_cast<int>(q[8]), static_cast<int>((unit_mask >> i) & 1)};
    if (!float_kind(r.run[i].dst_dt)) return DN_ERR_DTYPE;
    if (r.run[i].dims % 2 != 0 || r.run[i].dims < 0 || r.run[i].dims > r.run[i].width || r.run[i].n_vec < 0) return DN_ERR_SHAPE;
    if (unit_mask && r.run[i].width > 256) return DN_ERR_SHAPE;      // (a wave holds a vector of up to 256 numbers)
    vectors += r.run[i].n_vec;
  }
  if (T == 0) return 0;
  if (unit_mask) {
    if (vectors == 0 || (vectors + 3) / 4 > 65535) return vectors == 0 ? 0 : DN_ERR_SHAPE;
    hipLaunchKernelGGL(rotary_runs_unit_kernel, dim3(T, (vectors + 3) / 4), dim3(256), 0, stream, src, src_dt, static_cast<size_t>(ld_src), r,
                       positions, freq, mag, eps);
    return dn_launch_status();
  }
  hipLaunchKernelGGL(rotary_runs_kernel, dim3(T), dim3(256), 0, stream, src, src_dt, static_cast<size_t>(ld_src), r, positions, freq, mag);
  return dn_launch_status();
}

int dn_history_update(const void* h, int h_dt, long long ldh, float* hist, const int* row_start, const int* slots, int S, int width,
                      int keep, long long hist_stride, hipStream_t stream) {
  if (!float_kind(h_dt)) return DN_ERR_DTYPE;
  if (ldh < width) return DN_ERR_SHAPE;
  if (S == 0 || keep == 0) return 0;
  hipLaunchKernelGGL(history_update_kernel, dim3(S), dim3(256), 0, stream, h, h_dt, static_cast<size_t>(ldh), hist, row_start, slots, width, keep,
                     static_cast<size_t>(hist_stride));
  return dn_launch_status();
}

int dn_shift_mix(const void* h, int h_dt, const float* hist, const float* mu, int n_mix, const int* row_start, const int* slots, int S,
                 int T, int width, void* out, int out_dt, long long hist_stride, hipStream_t stream) {
  if (!float_kind(h_dt) || !float_kind(out_dt)) return DN_ERR_DTYPE;
  if (S < 1) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(shift_mix_kernel, dim3(T), dim3(256), 0, stream, h, h_dt, hist, mu, n_mix, row_start, slots, S, T, width, out,
                     out_dt, static_cast<size_t>(hist_stride));
  return dn_launch_status();
}

int dn_rotary(const void* src, int src_dt, long long ld_src, int src_off, int src_stride, void* dst, int dst_dt, long long ld_dst,
              int dst_off, int dst_stride, const int* positions, const float* freq, int T, int n_vec, int dims, int width, float mag,
              hipStream_t stream) {
  if (!float_kind(src_dt) || !float_kind(dst_dt)) return DN_ERR_DTYPE;
  if (dims % 2 != 0 || dims > width || dims < 0) return DN_ERR_SHAPE;
  if (T == 0 || n_vec == 0) return 0;
  hipLaunchKernelGGL(rotary_kernel, dim3(T), dim3(256), 0, stream, src, src_dt, static_cast<size_t>(ld_src), src_off, src_stride, dst,
                     dst_dt, static_cast<size_t>(ld_dst), dst_off, dst_stride, positions, freq, n_vec, dims, width, mag);
  return dn_launch_status();
}

int dn_activate(const float* x, long long ldx, const float* bias, const float* lower, int kind, void* out, int out_dt, long long ldo,
                int T, int n, hipStream_t stream) {
  if (!float_kind(out_dt)) return DN_ERR_DTYPE;
  if (kind < 0 || kind > ACT_RELU2 || ((kind == ACT_XIELU || kind == ACT_EXP_NEG_SOFTPLUS) && !lower)) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(activate_kernel, dim3(T), dim3(256), 0, stream, x, static_cast<size_t>(ldx), bias, lower, kind, out, out_dt,
                     static_cast<size_t>(ldo), n);
  return dn_launch_status();
}

int dn_gated(const void* x, int x_dt, long long ldx, const float* g, long long ldg, int kind, void* out, int out_dt, long long ldo,
             int T, int n, hipStream_t stream) {
  if (!float_kind(x_dt) || !float_kind(out_dt)) return DN_ERR_DTYPE;
  if (kind < 0 || kind > ACT_TANH) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(gated_kernel, dim3(T), dim3(256), 0, stream, x, x_dt, static_cast<size_t>(ldx), g, static_cast<size_t>(ldg), kind,
                     out, out_dt, static_cast<size_t>(ldo), n);
  return dn_launch_status();
}

int dn_state_scan(const float* r, long long ldr, const float* k, long long ldk, const float* v, long long ldv, const float* w,
                  long long ldw, const float* u, const float* beta, long long ldb, const float* w_head, int G, float* state,
                  long long slot_stride, const int* row_start, const int* slots, int S, int T, int H, int dk, int dv, int mode,
                  int key_from_decay, int beta_logits, int w_rows, float* out, long long ldo, hipStream_t stream) {
  if (dk < 1 || dk > 256 || dv < 1 || H < 1 || G < 1 || H % G != 0) return DN_ERR_SHAPE;
  if ((!key_from_decay && k == nullptr) || (w_rows && (w == nullptr || key_from_decay))) return DN_ERR_SHAPE;
  if (mode < SCAN_BEFORE || mode > SCAN_DELTA || (mode == SCAN_DELTA && beta == nullptr) || (w == nullptr) == (w_head == nullptr))
    return DN_ERR_SHAPE;
  if (S == 0) return 0;
  const int read_after = mode;
  ScanArgs a{r, k, v, w, u, beta, w_head, static_cast<size_t>(ldr), static_cast<size_t>(ldk), static_cast<size_t>(ldv),
             static_cast<size_t>(ldw), static_cast<size_t>(ldb), G, state, static_cast<size_t>(slot_stride), row_start, slots, H, dk, dv, read_after, key_from_decay, beta_logits, w_rows, out,
             static_cast<size_t>(ldo)};
  // (the parts of a column's sum by the head's size alone, never by the step: a row's bits are the same in every step)
  const dim3 few((dv + 15) / 16, H, S), many((dv + 3) / 4, H, S);
  auto by16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = dk % 4 == 0 && dv % 4 == 0 && ldr % 4 == 0 && ldv % 4 == 0 && (w == nullptr || w_rows || ldw % 4 == 0) &&
                   (key_from_decay || ldk % 4 == 0) && by16(r) && by16(v) && (w_rows || by16(w)) && (key_from_decay || by16(k));
  const bool few_rows = T <= 2 * S;      // (decoded tokens: a row or two a request)
#define DN_SCAN3(DK, KG, GRID, AFTER, VEC)                                                                    \
  do {                                                                                                        \
    if (few_rows) hipLaunchKernelGGL((scan_kernel<DK, KG, AFTER, VEC, 2>), GRID, dim3(64), 0, stream, a);  \
    else hipLaunchKernelGGL((scan_kernel<DK, KG, AFTER, VEC, (VEC ? 16 : 8)>), GRID, dim3(64), 0, stream, a); \
  } while (0)
#define DN_SCAN2(DK, KG, GRID, AFTER)        \
  do {                                       \
    if (vec) DN_SCAN3(DK, KG, GRID, AFTER, true); \
    else DN_SCAN3(DK, KG, GRID, AFTER, false);    \
  } while (0)
#define DN_SCAN(DK, KG, GRID)                                     \
  do {                                                            \
    if (mode == SCAN_DELTA) DN_SCAN2(DK, KG, GRID, SCAN_DELTA);   \
    else if (mode == SCAN_AFTER) DN_SCAN2(DK, KG, GRID, SCAN_AFTER); \
    else DN_SCAN2(DK, KG, GRID, SCAN_BEFORE);                     \
  } while (0)
  // (fewer lanes a column for long keys, so that fewer waves of a head fetch the same r, k and w, was measured on a model
  // of 32 heads with 128 channels x 64 columns and is slower: 2 x 1,024 rows 402 us at sixteen lanes, 469 at eight, 626 at
  // four; a row's chain of dependent sums grows with a lane's share of the column)
  if (dk <= 16) DN_SCAN(16, 4, few);
  else if (dk <= 32) DN_SCAN(32, 4, few);
  else if (dk <= 64) DN_SCAN(64, 16, many);
  else if (dk <= 128) DN_SCAN(128, 16, many);
  else DN_SCAN(256, 16, many);
#undef DN_SCAN2
#undef DN_SCAN3
#undef DN_SCAN
  return dn_launch_status();
}

int dn_head_norm(const float* o, long long ld, const float* weight, int w_stride, float eps, const float* gate, long long ldg,
                 int gate_kind, int gate_first, const float* skip, long long lds, const float* skip_scale, int skip_dim, void* out,
                 int out_dt, long long ldo, int T, int H, int dv, hipStream_t stream) {
  if (!float_kind(out_dt)) return DN_ERR_DTYPE;
  if (gate && (gate_kind < 0 || gate_kind > ACT_TANH)) return DN_ERR_SHAPE;
  if (skip && (!skip_scale || skip_dim < 1)) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  HeadNormArgs a{o, static_cast<size_t>(ld), weight, w_stride, eps, gate, static_cast<size_t>(ldg), gate_kind, gate_first, skip,
                 static_cast<size_t>(lds), skip_scale, skip_dim, out, out_dt, static_cast<size_t>(ldo), dv};
  if (dv > 256 && dv <= 2048)
    hipLaunchKernelGGL(head_norm_held_kernel<8>, dim3(T, H), dim3(256), 0, stream, a);
  else if (dv > 2048 && dv <= 4096)
    hipLaunchKernelGGL(head_norm_held_kernel<16>, dim3(T, H), dim3(256), 0, stream, a);
  else if (dv > 256)
    hipLaunchKernelGGL(head_norm_wide_kernel, dim3(T, H), dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL(head_norm_kernel, dim3(T, H), dim3(64), 0, stream, a);
  return dn_launch_status();
}

int dn_step_sizes(const float* z, long long ldz, const float* bias, const float* rate, const float* x, long long ldx, int T, int H, int dv,
                  float* decay, long long ldd, float* v, long long ldv, hipStream_t stream) {
  if (H < 1 || dv < 1 || !rate) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(step_sizes_kernel, dim3(T), dim3(256), 0, stream, z, static_cast<size_t>(ldz), bias, rate, x, static_cast<size_t>(ldx),
                     H, dv, decay, static_cast<size_t>(ldd), v, static_cast<size_t>(ldv));
  return dn_launch_status();
}

int dn_gate_scan(const float* a, long long lda, const float* b, long long ldb, const float* g, long long ldg, const float* bias_a,
                 const float* bias_b, float* state, long long slot_stride, const int* row_start, const int* slots, int S, int T, int width,
                 void* out, int out_dt, long long ldo, hipStream_t stream) {
  if (!float_kind(out_dt)) return DN_ERR_DTYPE;
  if (width < 1 || S > 65535) return DN_ERR_SHAPE;
  if (S == 0) return 0;
  // (decoded tokens, a row or two a request: one wave; portions: sixteen waves of eight rows each at a time)
  if (T <= 2 * S)
    hipLaunchKernelGGL(gate_scan_kernel<1>, dim3((width + 63) / 64, S), dim3(64), 0, stream, a, static_cast<size_t>(lda), b,
                       static_cast<size_t>(ldb), g, static_cast<size_t>(ldg), bias_a, bias_b, state, static_cast<size_t>(slot_stride),
                       row_start, slots, width, out, out_dt, static_cast<size_t>(ldo));
  else
    hipLaunchKernelGGL(gate_scan_kernel<16>, dim3((width + 63) / 64, S), dim3(1024), 0, stream, a, static_cast<size_t>(lda), b,
                       static_cast<size_t>(ldb), g, static_cast<size_t>(ldg), bias_a, bias_b, state, static_cast<size_t>(slot_stride),
                       row_start, slots, width, out, out_dt, static_cast<size_t>(ldo));
  return dn_launch_status();
}

int dn_streams_read(const float* xs, long long plane, int n, const float* w_in, const float* g, float eps, void* out, int out_dt,
                    long long ldo, const int* rows, int R, int width, hipStream_t stream) {
  if (!float_kind(out_dt)) return DN_ERR_DTYPE;
  if (n < 1 || n > STREAMS_MAX || width < 1) return DN_ERR_SHAPE;
  if (R == 0) return 0;
  hipLaunchKernelGGL(streams_read_kernel, dim3(R), dim3(256), 0, stream, xs, static_cast<size_t>(plane), n, w_in, g, eps, out, out_dt,
                     static_cast<size_t>(ldo), rows, width);
  return dn_launch_status();
}

int dn_streams_write(float* xs, long long plane, int n, const float* mix, const float* w_out, const float* y, long long ldy,
                     const float* y2, long long ldy2, const float* by, const float* by2, float beps, const float* next_in,
                     const float* g, float eps, void* out, int out_dt, long long ldo, int T, int width, hipStream_t stream) {
  if (next_in && !float_kind(out_dt)) return DN_ERR_DTYPE;
  if (n < 1 || n > STREAMS_MAX || width < 1 || (next_in && !out) || (y2 && (!by || !by2))) return DN_ERR_SHAPE;
  if (T == 0) return 0;
#define DN_STREAMS_HELD(NS, NC)                                                                                              \
  hipLaunchKernelGGL((streams_write_held_kernel<NS, NC>), dim3(T), dim3(256), 0, stream, xs, static_cast<size_t>(plane), n, mix,    \
                     w_out, y, static_cast<size_t>(ldy), y2, static_cast<size_t>(ldy2), by, by2, beps, next_in, g, eps, out, out_dt, \
                     static_cast<size_t>(ldo), width)
  // (up to 4 copies of rows up to 4,096 wide: a thread holds its share of the row; by the sizes alone, the same bits either way)
  if (n <= 2 && width <= 1024) DN_STREAMS_HELD(2, 4);
  else if (n <= 2 && width <= 2048) DN_STREAMS_HELD(2, 8);
  else if (n <= 4 && width <= 1024) DN_STREAMS_HELD(4, 4);
  else if (n <= 4 && width <= 2048) DN_STREAMS_HELD(4, 8);
  else if (n <= 4 && width <= 4096) DN_STREAMS_HELD(4, 16);
  else
    hipLaunchKernelGGL(streams_write_kernel, dim3(T), dim3(256), 0, stream, xs, static_cast<size_t>(plane), n, mix, w_out, y,
                       static_cast<size_t>(ldy), y2, static_cast<size_t>(ldy2), by, by2, beps, next_in, g, eps, out, out_dt,
                       static_cast<size_t>(ldo), width);
#undef DN_STREAMS_HELD
  return dn_launch_status();
}

int dn_norm_pair_write(const float* z, long long ldz, int qw, int kw, const float* wq, const float* wk, float eps, void* q_out,
                       long long ldq, const int* slot_map, void* k_pool, void* v_pool, int T, int Hkv, int dh, int page_size,
                       int dt, int write, hipStream_t stream) {
  if (!float_kind(dt)) return DN_ERR_DTYPE;
  if (qw < 1 || kw != Hkv * dh || page_size < 1 || ldz < qw + kw || ldq < qw) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(norm_pair_write_kernel, dim3(T), dim3(256), 0, stream, z, static_cast<size_t>(ldz), qw, kw, wq, wk, eps, q_out,
                     static_cast<size_t>(ldq), slot_map, k_pool, v_pool, dh, page_size, dt, write);
  return dn_launch_status();
}

int dn_head_gate(const void* o, int o_dt, long long ldo, int head_stride, const float* g, long long ldg, void* out, int out_dt,
                 long long ldout, int T, int n_heads, int dv, hipStream_t stream) {
  if (!float_kind(o_dt) || !float_kind(out_dt)) return DN_ERR_DTYPE;
  if (n_heads < 1 || dv < 1 || head_stride < dv || ldg < n_heads) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(head_gate_kernel, dim3(T), dim3(256), 0, stream, o, o_dt, static_cast<size_t>(ldo), head_stride, g,
                     static_cast<size_t>(ldg), out, out_dt, static_cast<size_t>(ldout), n_heads, dv);
  return dn_launch_status();
}

int dn_rows_times_table(const void* a, int a_dt, long long lda, const void* table, int t_dt, long long ldt, int off, const int* ids,
                        int n_rows, void* out, int out_dt, long long ldo, int T, int n, hipStream_t stream) {
  if (!float_kind(a_dt) || !float_kind(t_dt) || !float_kind(out_dt)) return DN_ERR_DTYPE;
  if (n < 1 || off < 0 || off + n > ldt || n_rows < 1) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  hipLaunchKernelGGL(rows_times_table_kernel, dim3(T), dim3(256), 0, stream, a, a_dt, static_cast<size_t>(lda), table, t_dt,
                     static_cast<size_t>(ldt), off, ids, n_rows, out, out_dt, static_cast<size_t>(ldo), n);
  return dn_launch_status();
}

int dn_selective_scan(const void* x, int x_dt, long long ldx, const float* dt, long long ldd, const float* dt_bias, const float* B, long long ldb,
                      const float* C, long long ldc, const float* A, const float* D, const float* z, long long ldz, float* state,
                      long long slot_stride, const int* row_start, const int* slots, int S, int T, int inner, int N, void* out,
                      int out_dt, long long ldo, int in_order, hipStream_t stream) {
  if (!float_kind(out_dt) || !float_kind(x_dt)) return DN_ERR_DTYPE;
  if (inner < 1 || N < 1 || N > 256 || S > 65535 || slot_stride < static_cast<long long>(inner) * N) return DN_ERR_SHAPE;
  if (S == 0) return 0;
  const SelectiveArgs a{x, x_dt, dt, dt_bias, B, C, A, D, z, static_cast<size_t>(ldx), static_cast<size_t>(ldd), static_cast<size_t>(ldb),
                        static_cast<size_t>(ldc), static_cast<size_t>(ldz), state, static_cast<size_t>(slot_stride), row_start, slots,
                        inner, N, out, out_dt, static_cast<size_t>(ldo)};
  const int per = (N + 15) / 16;
  // (portions of few requests: the rows shared out among eight waves, which leaves a wave the registers of half a SIMD; up to four states a lane)
  if (!in_order && per <= 4 && T > 32 * S && static_cast<long long>(S) * ((inner + 15) / 16) < 2048) {
    const dim3 runs((inner + 3) / 4, S);
    if (per <= 1) hipLaunchKernelGGL((selective_scan_runs_kernel<1, 8, 8>), runs, dim3(512), 0, stream, a);
    else if (per <= 2) hipLaunchKernelGGL((selective_scan_runs_kernel<2, 8, 4>), runs, dim3(512), 0, stream, a);
    else hipLaunchKernelGGL((selective_scan_runs_kernel<4, 8, 2>), runs, dim3(512), 0, stream, a);
    return dn_launch_status();
  }
  if (T <= 2 * S && per <= 2 && static_cast<long long>(S) * ((inner + 15) / 16) >= 2048) {
    // a step of single rows of many requests (more workgroups of 16 channels than the chip holds at a time): a lane takes
    // four channels, their loads in flight together (batch 64, 2,048 channels: 38 -> 29 us; at batch 8 it is no faster)
    const dim3 few((inner + 63) / 64, S);
    if (per <= 1) hipLaunchKernelGGL((selective_scan_kernel<1, 4, 1>), few, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((selective_scan_kernel<2, 4, 1>), few, dim3(256), 0, stream, a);
    return dn_launch_status();
  }
  const dim3 grid((inner + 15) / 16, S);
  if (per <= 1) hipLaunchKernelGGL((selective_scan_kernel<1, 1, 4>), grid, dim3(256), 0, stream, a);
  else if (per <= 2) hipLaunchKernelGGL((selective_scan_kernel<2, 1, 4>), grid, dim3(256), 0, stream, a);
  else if (per <= 4) hipLaunchKernelGGL((selective_scan_kernel<4, 1, 2>), grid, dim3(256), 0, stream, a);
  else if (per <= 8) hipLaunchKernelGGL((selective_scan_kernel<8, 1, 1>), grid, dim3(256), 0, stream, a);
  else hipLaunchKernelGGL((selective_scan_kernel<16, 1, 1>), grid, dim3(256), 0, stream, a);
  return dn_launch_status();
}

int dn_token_input(float* x, long long ldx, const void* wg, const void* wp, int w_dt, const void* table, int t_dt, long long ldt, int off,
                   const int* ids, int n_rows, const float* weight, int T, int width, int dim, float eps, const float* next_w,
                   float next_eps, void* next_out, int next_dt, long long ldn, hipStream_t stream) {
  if (!float_kind(w_dt) || !float_kind(t_dt) || (next_out && (!float_kind(next_dt) || ldn < width))) return DN_ERR_DTYPE;
  if (width < 1 || dim < 1 || off < 0 || off + dim > ldt || n_rows < 1 || (2 * static_cast<long long>(width) + dim) * 4 > 60000) return DN_ERR_SHAPE;
  if (T == 0) return 0;
  const size_t lds = (2 * static_cast<size_t>(width) + dim) * sizeof(float);
  const bool vec = w_dt == DN_BF16 && width % 8 == 0 && dim % 8 == 0 && reinterpret_cast<uintptr_t>(wg) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(wp) % 16 == 0;
  if (vec)
    hipLaunchKernelGGL(token_input_kernel<true>, dim3(T), dim3(1024), lds, stream, x, static_cast<size_t>(ldx), wg, wp, w_dt, table, t_dt,
                       static_cast<size_t>(ldt), off, ids, n_rows, weight, width, dim, eps, next_w, next_eps, next_out, next_dt,
                       static_cast<size_t>(ldn));
  else
    hipLaunchKernelGGL(token_input_kernel<false>, dim3(T), dim3(1024), lds, stream, x, static_cast<size_t>(ldx), wg, wp, w_dt, table, t_dt,
                       static_cast<size_t>(ldt), off, ids, n_rows, weight, width, dim, eps, next_w, next_eps, next_out, next_dt,
                       static_cast<size_t>(ldn));
  return dn_launch_status();
}

}  // extern "C"
