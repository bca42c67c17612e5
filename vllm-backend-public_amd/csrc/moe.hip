// Mixture-of-experts feed-forward: routing, the expert-sorted row order, and the expert products for
// steps of few rows.
//   moe_route           scores from fp32 router logits (a sigmoid each, a softmax over all of them, or the
//                       logits themselves with a softmax over the chosen ones as weights);
//                       experts are picked by score + correction among the experts of the best `keep` of
//                       `count` groups of neighbours (a group scores the sum of its two best, or its
//                       best), and weighted by the score without correction, times a constant
//   moe_sort            rows (token, choice) ordered by expert: offsets[E + 1], perm[position] = row,
//                       inv[row] = position
//   moe_gather_rows     xs[position] = x[perm[position] / top]; or every expert's rows padded to a common count
//   moe_gate_up_rows    a[position] = silu(Wg[e] x) * (Wu[e] x) for every routed row, one wave per
//                       (expert, hidden unit) walking that expert's rows: an expert's weights leave HBM once
//   moe_down_rows       y[position] = Wd[e] a[position], the same way; both on the matrix cores where the
//                       sizes allow (16-bit storage, widths multiples of 32 / 16)
//   moe_silu_and_mul    a = silu(gu[:, :F]) * gu[:, F:] (any storage type)
//   moe_combine         out[t] = sum_k weight[t, k] * y[inv[t * top + k]]; a chosen id at or past `num_real`
//                       is an identity expert and stands for x[t]; a shared expert's rows join, times the
//                       sigmoid of one fp32 number per token
// The gated activation of an expert is silu(g) * u, or (act 1) with g = min(g, limit) and
// u = clamp(u, -limit, limit): g * sigmoid(1.702 g) * (u + 1).
// Routing, scores and the weighted sum are fp32; activations and expert weights are stored in the
// dtype argument's type, products accumulate in fp32.
#include "common.h"

namespace mi355 {

constexpr int kMaxGroups = 64;
constexpr int kMaxTop = 16;

// softmax == 2: the stored weights are the chosen logits; they become a softmax over the chosen
// alone, times wscale.  The thread that stored them rewrites them.
__device__ __forceinline__ void chosen_softmax(float* w, [[maybe_unused]] const float* base, int top, float wscale) {
  float mx = -__builtin_inff();
  for (int r = 0; r < top; ++r) mx = fmaxf(mx, MI355_LD(float, base, w + r));
  float sum = 0.f;
  for (int r = 0; r < top; ++r) sum += expf(MI355_LD(float, base, w + r) - mx);
  for (int r = 0; r < top; ++r) MI355_ST(float, base, w + r, expf(MI355_LD(float, base, w + r) - mx) / sum * wscale);
}

__global__ __launch_bounds__(64) void moe_route_kernel(int32_t* __restrict__ ids, float* __restrict__ wts,
                                                       const float* __restrict__ z, int64_t z_stride,
                                                       const float* __restrict__ corr, int64_t T, int E, int top, int count,
                                                       int keep, int softmax, int group_max, float wscale) {
  const int64_t t = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (t >= T) return;
  const float* zr = z + t * z_stride;
  const int per = E / count;
  const float ninf = -__builtin_inff();
  float zmax = ninf, zsum = 1.0f;
  if (softmax == 1) {
    for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, MI355_LD(float, z, zr + e));
    zsum = 0.f;
    for (int e = 0; e < E; ++e) zsum += expf(MI355_LD(float, z, zr + e) - zmax);
  }
  auto score = [&](int e) {
    const float v = MI355_LD(float, z, zr + e);
    return softmax == 2 ? v : softmax ? expf(v - zmax) / zsum : 1.0f / (1.0f + expf(-v));
  };
  auto choice = [&](int e) { return score(e) + MI355_LD(float, corr, corr + e); };
  // the groups that stay: `keep` rounds of picking the best group not yet picked
  uint64_t allowed = 0;
  if (keep >= count) {
    allowed = ~0ull;
  } else {
    for (int r = 0; r < keep; ++r) {
      int best = -1;
      float bs = ninf;
      for (int g = 0; g < count; ++g) {
        if ((allowed >> g) & 1ull) continue;
        float a = ninf, b = ninf;                       // the two largest of the group
        for (int i = 0; i < per; ++i) {
          const float c = choice(g * per + i);
          if (c > a) { b = a; a = c; } else if (c > b) { b = c; }
        }
        const float gs = (per > 1 && !group_max) ? a + b : a;
        if (best < 0 || gs > bs) { best = g; bs = gs; }
      }
      allowed |= 1ull << best;
    }
  }
  int picked[kMaxTop];
  for (int r = 0; r < top; ++r) {
    int best = -1;
    float bs = ninf;
    for (int e = 0; e < E; ++e) {
      if (!((allowed >> (e / per)) & 1ull)) continue;
      bool taken = false;
      for (int q = 0; q < r; ++q) taken |= picked[q] == e;
      if (taken) continue;
      const float c = choice(e);
      if (best < 0 || c > bs) { best = e; bs = c; }
    }
    picked[r] = best;
    MI355_ST(int32_t, ids, ids + t * top + r, best);
    MI355_ST(float, wts, wts + t * top + r, score(best) * (softmax == 2 ? 1.0f : wscale));
  }
  if (softmax == 2) chosen_softmax(wts + t * top, wts, top, wscale);
}

// (value, index) maximum over the wave, every lane gets it; ties go to the lower index
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, 64);
    const int oi = __shfl_xor(i, off, 64);
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
  }
}

// The same choice, one wave per token: lane j holds experts j, j + 64, ...; groups are scored by the
// lanes from the choice scores in LDS; every pick is a maximum over the wave.
template <int EPL>
__global__ __launch_bounds__(256) void moe_route_wave_kernel(int32_t* __restrict__ ids, float* __restrict__ wts,
                                                             const float* __restrict__ z, int64_t z_stride,
                                                             const float* __restrict__ corr, int64_t T, int E, int top,
                                                             int count, int keep, int softmax, int group_max, float wscale) {
  __shared__ float ch[4][64 * EPL];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int64_t t = blockIdx.x * 4 + wave;
  const bool live = t < T;
  if (!live) t = T - 1;                                 // (every wave reaches the barrier; nothing stored)
  const float* zr = z + t * z_stride;
  const float ninf = -__builtin_inff();
  const int per = E / count;
  float zmax = ninf, zsum = 1.0f;
  if (softmax == 1) {                                   // over all router outputs, in fp32
#pragma unroll
    for (int i = 0; i < EPL; ++i)
      if (lane + 64 * i < E) zmax = fmaxf(zmax, MI355_LD(float, z, zr + lane + 64 * i));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) zmax = fmaxf(zmax, __shfl_xor(zmax, off, 64));
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i)
      if (lane + 64 * i < E) part += expf(MI355_LD(float, z, zr + lane + 64 * i) - zmax);
    zsum = wave_sum(part);
  }
  auto score = [&](int e) {
    const float v = MI355_LD(float, z, zr + e);
    return softmax == 2 ? v : softmax ? expf(v - zmax) / zsum : 1.0f / (1.0f + expf(-v));
  };
  float c[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + 64 * i;
    c[i] = e < E ? score(e) + MI355_LD(float, corr, corr + e) : ninf;
    if (c[i] != c[i]) c[i] = -3.0e38f;                  // a NaN logit ranks last but stays a valid pick: ids are indices downstream
    ch[wave][e] = c[i];
  }
  __syncthreads();
  if (keep < count) {
    float gs = ninf;
    if (lane < count) {
      float a = ninf, b = ninf;                         // the two largest of the group
      for (int i = 0; i < per; ++i) {
        const float v = ch[wave][lane * per + i];
        if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
      }
      gs = (per > 1 && !group_max) ? a + b : a;
    }
    uint64_t allowed = 0;
    bool mine = false;                                  // this lane's group has been picked
    for (int r = 0; r < keep; ++r) {
      float v = (lane < count && !mine) ? gs : ninf;
      int g = (lane < count && !mine) ? lane : 0x7FFFFFFF;
      wave_argmax(v, g);
      if (lane == g) mine = true;
      allowed |= 1ull << g;
    }
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int e = lane + 64 * i;
      if (e < E && !((allowed >> (e / per)) & 1ull)) c[i] = ninf;
    }
  }
  for (int r = 0; r < top; ++r) {
    float v = ninf;
    int e = 0x7FFFFFFF;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int ei = lane + 64 * i;
      if (ei < E && (c[i] > v || e == 0x7FFFFFFF) && c[i] > ninf) { v = c[i]; e = ei; }
    }
    wave_argmax(v, e);
#pragma unroll
    for (int i = 0; i < EPL; ++i)
      if (lane + 64 * i == e) c[i] = ninf;              // taken
    if (live && lane == 0) {
      MI355_ST(int32_t, ids, ids + t * top + r, e);
      MI355_ST(float, wts, wts + t * top + r, score(e) * (softmax == 2 ? 1.0f : wscale));
    }
  }
  if (softmax == 2 && live && lane == 0) chosen_softmax(wts + t * top, wts, top, wscale);
}

// one workgroup: counts, an exclusive prefix, then a position for every row
__global__ __launch_bounds__(1024) void moe_sort_kernel(int32_t* __restrict__ offsets, int32_t* __restrict__ perm,
                                                        int32_t* __restrict__ inv, const int32_t* __restrict__ ids,
                                                        int64_t rows, int E) {
  extern __shared__ int32_t sm[];                       // counts [E] | starts [E + 1]
  int32_t* cnt = sm;
  int32_t* start = sm + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) atomicAdd(&cnt[MI355_LD(int32_t, ids, ids + r)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t at = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      at += cnt[e];
    }
    start[E] = at;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += blockDim.x) MI355_ST(int32_t, offsets, offsets + e, start[e]);
  __syncthreads();
  // positions inside an expert's range are handed out in arrival order: which row lands where varies
  // from run to run, what is computed for a row does not depend on it
  for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) {
    const int32_t at = atomicAdd(&start[MI355_LD(int32_t, ids, ids + r)], 1);
    MI355_ST(int32_t, perm, perm + at, static_cast<int32_t>(r));
    MI355_ST(int32_t, inv, inv + r, at);
  }
}

// cap 0: xs[position] for every routed row.  cap > 0: every expert's rows padded to cap, xs[e * cap + j]
// = the j-th row of expert e, zeros past its count (grid: experts * cap rows)
template <typename T>
__global__ __launch_bounds__(256) void moe_gather_rows_kernel(typename Elem<T>::S* __restrict__ xs,
                                                              const typename Elem<T>::S* __restrict__ x,
                                                              const int32_t* __restrict__ perm,
                                                              const int32_t* __restrict__ offsets, int cap, int top, int W) {
  int64_t p = blockIdx.x;
  bool have = true;
  if (cap > 0) {
    const int e = static_cast<int>(p / cap), j = static_cast<int>(p % cap);
    const int lo = MI355_LD(int32_t, offsets, offsets + e), hi = MI355_LD(int32_t, offsets, offsets + e + 1);
    have = j < hi - lo;
    p = lo + j;
  }
  const int64_t t = have ? MI355_LD(int32_t, perm, perm + p) / top : 0;
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    MI355_ST(typename Elem<T>::S, xs, xs + static_cast<int64_t>(blockIdx.x) * W + c,
             have ? MI355_LD(typename Elem<T>::S, x, x + t * W + c) : typename Elem<T>::S(0));
}

__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + expf(-g)); }

// the gated activation of an expert (see the head of this file)
__device__ __forceinline__ float gated_act(float g, float u, int act, float limit) {
  if (act == 0) return silu_f(g) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
}

// Rows of an expert are taken kRowBlock at a time, so that a weight element is loaded once per block
// of rows and not once per row.
constexpr int kRowBlock = 8;

// dot products of one weight row w [n] with up to kRowBlock rows xr[r] [n]; every lane of the wave gets the sums
template <typename T, bool VEC>
__device__ __forceinline__ void rows_dot(const typename Elem<T>::S* wbase, const typename Elem<T>::S* w,
                                         const typename Elem<T>::S* xbase, const typename Elem<T>::S* const (&xr)[kRowBlock],
                                         int n, int lane, float (&acc)[kRowBlock]) {
#pragma unroll
  for (int r = 0; r < kRowBlock; ++r) acc[r] = 0.f;
  if constexpr (VEC) {                                  // 16-bit storage, n a multiple of 8, 16-byte aligned rows
    for (int c = lane * 8; c < n; c += 512) {
      float wv[8];
      unpack8<T>(MI355_LD(uint4, wbase, reinterpret_cast<const uint16_t*>(w) + c), wv);
#pragma unroll
      for (int r = 0; r < kRowBlock; ++r) {
        float xv[8];
        unpack8<T>(MI355_LD(uint4, xbase, reinterpret_cast<const uint16_t*>(xr[r]) + c), xv);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[r] += wv[i] * xv[i];
      }
    }
  } else {
    for (int c = lane; c < n; c += 64) {
      const float wv = MI355_LDF(T, wbase, w + c);
#pragma unroll
      for (int r = 0; r < kRowBlock; ++r) acc[r] += wv * MI355_LDF(T, xbase, xr[r] + c);
    }
  }
#pragma unroll
  for (int r = 0; r < kRowBlock; ++r) acc[r] = wave_sum(acc[r]);
}

template <typename T, bool VEC> struct RowsDot {
  static __device__ __forceinline__ void run(const typename Elem<T>::S* wbase, const typename Elem<T>::S* w,
                                             const typename Elem<T>::S* xbase,
                                             const typename Elem<T>::S* const (&xr)[kRowBlock], int n, int lane,
                                             float (&acc)[kRowBlock]) {
    rows_dot<T, VEC>(wbase, w, xbase, xr, n, lane, acc);
  }
};
template <> struct RowsDot<F32, true> {                  // (never selected: 32-bit storage takes the scalar form)
  static __device__ __forceinline__ void run(const float* wbase, const float* w, const float* xbase,
                                             const float* const (&xr)[kRowBlock], int n, int lane, float (&acc)[kRowBlock]) {
    rows_dot<F32, false>(wbase, w, xbase, xr, n, lane, acc);
  }
};

// one wave per (expert, hidden unit f): gate and up rows of that unit against every row routed to the expert
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void moe_gate_up_rows_kernel(typename Elem<T>::S* __restrict__ a,
                                                               const typename Elem<T>::S* __restrict__ x,
                                                               const typename Elem<T>::S* __restrict__ w_gate_up,
                                                               const int32_t* __restrict__ offsets,
                                                               const int32_t* __restrict__ perm, int top, int W, int F,
                                                               int act, float limit) {
  typedef typename Elem<T>::S E;
  const int e = blockIdx.y, lane = threadIdx.x & 63;
  const int f = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (f >= F) return;
  const int lo = MI355_LD(int32_t, offsets, offsets + e), hi = MI355_LD(int32_t, offsets, offsets + e + 1);
  const E* wg = w_gate_up + (static_cast<int64_t>(e) * 2 * F + f) * W;
  const E* wu = wg + static_cast<int64_t>(F) * W;
  for (int p0 = lo; p0 < hi; p0 += kRowBlock) {
    const E* xr[kRowBlock];
#pragma unroll
    for (int r = 0; r < kRowBlock; ++r) {                // rows past the expert's last: the block's first row again, not stored
      const int p = p0 + r < hi ? p0 + r : p0;
      xr[r] = x + static_cast<int64_t>(MI355_LD(int32_t, perm, perm + p) / top) * W;
    }
    float g[kRowBlock], u[kRowBlock];
    RowsDot<T, VEC>::run(w_gate_up, wg, x, xr, W, lane, g);
    RowsDot<T, VEC>::run(w_gate_up, wu, x, xr, W, lane, u);
#pragma unroll
    for (int r = 0; r < kRowBlock; ++r) {
      if (lane == r && p0 + r < hi) {
        const float gr = elem_to_f<T>(elem_from_f<T>(g[r])), ur = elem_to_f<T>(elem_from_f<T>(u[r]));   // as stored by a product
        MI355_STF(T, a, a + static_cast<int64_t>(p0 + r) * F + f, gated_act(gr, ur, act, limit));
      }
    }
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void moe_down_rows_kernel(typename Elem<T>::S* __restrict__ y,
                                                            const typename Elem<T>::S* __restrict__ a,
                                                            const typename Elem<T>::S* __restrict__ w_down,
                                                            const int32_t* __restrict__ offsets, int W, int F) {
  typedef typename Elem<T>::S E;
  const int e = blockIdx.y, lane = threadIdx.x & 63;
  const int c = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (c >= W) return;
  const int lo = MI355_LD(int32_t, offsets, offsets + e), hi = MI355_LD(int32_t, offsets, offsets + e + 1);
  const E* wd = w_down + (static_cast<int64_t>(e) * W + c) * F;
  for (int p0 = lo; p0 < hi; p0 += kRowBlock) {
    const E* ar[kRowBlock];
#pragma unroll
    for (int r = 0; r < kRowBlock; ++r) ar[r] = a + static_cast<int64_t>(p0 + r < hi ? p0 + r : p0) * F;
    float s[kRowBlock];
    RowsDot<T, VEC>::run(w_down, wd, a, ar, F, lane, s);
#pragma unroll
    for (int r = 0; r < kRowBlock; ++r)
      if (lane == r && p0 + r < hi) MI355_STF(T, y, y + static_cast<int64_t>(p0 + r) * W + c, s[r]);
  }
}

// The same two products on the matrix cores (16-bit storage): a wave streams 16 weight rows of one
// expert once and multiplies them into that expert's routed rows, 16 at a time -- the rows are the
// columns of a 16 x 16 x 32 product, so a decode step's handful of rows per expert costs one pass
// over the expert's weights and one matrix instruction per 32 weights of a row.
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_mfma_kernel(uint16_t* __restrict__ a, const uint16_t* __restrict__ x,
                                                               const uint16_t* __restrict__ w_gate_up,
                                                               const int32_t* __restrict__ offsets,
                                                               const int32_t* __restrict__ perm, int top, int W, int F,
                                                               int act, float limit) {
  const int e = blockIdx.y, lane = threadIdx.x & 63, li = lane & 15, kk = lane >> 4;
  const int f0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 16;
  if (f0 >= F) return;
  const int lo = MI355_LD(int32_t, offsets, offsets + e), hi = MI355_LD(int32_t, offsets, offsets + e + 1);
  const uint16_t* wg = w_gate_up + (static_cast<int64_t>(e) * 2 * F + f0 + li) * W + 8 * kk;
  const uint16_t* wu = wg + static_cast<int64_t>(F) * W;
  for (int p0 = lo; p0 < hi; p0 += 16) {
    const int p = p0 + li < hi ? p0 + li : p0;          // columns past the expert's last row: its first row again, not stored
    const uint16_t* xr = x + static_cast<int64_t>(MI355_LD(int32_t, perm, perm + p) / top) * W + 8 * kk;
    f32x4 g = f32x4{0.f, 0.f, 0.f, 0.f}, u = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < W; s += 32) {                   // (two chains of products in turn: gate, up)
      const uint4 b = MI355_LD(uint4, x, xr + s);
      g = T::mfma(MI355_LD(uint4, w_gate_up, wg + s), b, g);
      u = T::mfma(MI355_LD(uint4, w_gate_up, wu + s), b, u);
    }
    if (p0 + li < hi) {
      float out[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) out[r] = gated_act(round_f<T>(g[r]), round_f<T>(u[r]), act, limit);      // as stored by a product
      MI355_ST(uint2, a, a + static_cast<int64_t>(p0 + li) * F + f0 + 4 * kk,
               make_uint2(T::pack2(out[0], out[1]), T::pack2(out[2], out[3])));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_mfma_kernel(uint16_t* __restrict__ y, const uint16_t* __restrict__ a,
                                                            const uint16_t* __restrict__ w_down,
                                                            const int32_t* __restrict__ offsets, int W, int F) {
  const int e = blockIdx.y, lane = threadIdx.x & 63, li = lane & 15, kk = lane >> 4;
  const int c0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 16;
  if (c0 >= W) return;
  const int lo = MI355_LD(int32_t, offsets, offsets + e), hi = MI355_LD(int32_t, offsets, offsets + e + 1);
  const uint16_t* wd = w_down + (static_cast<int64_t>(e) * W + c0 + li) * F + 8 * kk;
  for (int p0 = lo; p0 < hi; p0 += 16) {
    const uint16_t* ar = a + static_cast<int64_t>(p0 + li < hi ? p0 + li : p0) * F + 8 * kk;
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f}, acc2 = f32x4{0.f, 0.f, 0.f, 0.f};     // two chains of products in turn
    for (int s = 0; s < F; s += 64) {
      acc = T::mfma(MI355_LD(uint4, w_down, wd + s), MI355_LD(uint4, a, ar + s), acc);
      if (s + 32 < F) acc2 = T::mfma(MI355_LD(uint4, w_down, wd + s + 32), MI355_LD(uint4, a, ar + s + 32), acc2);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] += acc2[r];
    if (p0 + li < hi)
      MI355_ST(uint2, y, y + static_cast<int64_t>(p0 + li) * W + c0 + 4 * kk,
               make_uint2(T::pack2(acc[0], acc[1]), T::pack2(acc[2], acc[3])));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_silu_and_mul_kernel(typename Elem<T>::S* __restrict__ out,
                                                               const typename Elem<T>::S* __restrict__ x, int64_t rows,
                                                               int F, int act, float limit) {
  const int64_t total = rows * F;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / F;
    const int f = static_cast<int>(i % F);
    MI355_STF(T, out, out + i, gated_act(MI355_LDF(T, x, x + r * 2 * F + f), MI355_LDF(T, x, x + r * 2 * F + F + f), act, limit));
  }
}

// the same activation for rows whose gate and up parts are column slices of a wider buffer, into a
// column slice of another
template <typename T>
__global__ __launch_bounds__(256) void gated_act_rows_kernel(typename Elem<T>::S* __restrict__ out, int64_t out_stride,
                                                             const typename Elem<T>::S* __restrict__ gate,
                                                             const typename Elem<T>::S* __restrict__ up, int64_t in_stride,
                                                             int64_t rows, int F, int act, float limit) {
  const int64_t total = rows * F;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / F;
    const int f = static_cast<int>(i % F);
    MI355_STF(T, out, out + r * out_stride + f,
              gated_act(MI355_LDF(T, gate, gate + r * in_stride + f), MI355_LDF(T, up, up + r * in_stride + f), act, limit));
  }
}

// 16-bit storage, 8 hidden units per thread (ff a multiple of 8, rows and slices on 16-byte boundaries)
template <typename T>
__global__ __launch_bounds__(256) void gated_act_rows_vec_kernel(uint16_t* __restrict__ out, int64_t out_stride,
                                                                 const uint16_t* __restrict__ gate,
                                                                 const uint16_t* __restrict__ up, int64_t in_stride,
                                                                 int64_t rows, int F8, int act, float limit) {
  const int64_t total = rows * F8;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / F8;
    const int f = static_cast<int>(i % F8) * 8;
    const uint4 g4 = MI355_LD(uint4, gate, gate + r * in_stride + f);
    const uint4 u4 = MI355_LD(uint4, up, up + r * in_stride + f);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      o[j] = T::pack2(gated_act(T::to_f(static_cast<uint16_t>(gw[j] & 0xFFFFu)), T::to_f(static_cast<uint16_t>(uw[j] & 0xFFFFu)), act, limit),
                      gated_act(T::to_f(static_cast<uint16_t>(gw[j] >> 16)), T::to_f(static_cast<uint16_t>(uw[j] >> 16)), act, limit));
    MI355_ST(uint4, out, out + r * out_stride + f, make_uint4(o[0], o[1], o[2], o[3]));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(typename Elem<T>::S* __restrict__ out,
                                                          const typename Elem<T>::S* __restrict__ y,
                                                          const int32_t* __restrict__ inv, const float* __restrict__ wts,
                                                          const int32_t* __restrict__ ids,
                                                          const int32_t* __restrict__ offsets, int cap, int top, int W,
                                                          const typename Elem<T>::S* __restrict__ x, int num_real,
                                                          const typename Elem<T>::S* __restrict__ shared,
                                                          const float* __restrict__ shared_gate, int64_t shared_gate_stride) {
  const int64_t t = blockIdx.x;
  float sg = 0.f;
  if (shared != nullptr)
    sg = shared_gate != nullptr ? 1.0f / (1.0f + expf(-MI355_LD(float, shared_gate, shared_gate + t * shared_gate_stride))) : 1.0f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float s = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = ids != nullptr ? MI355_LD(int32_t, ids, ids + t * top + k) : 0;
      const float w = MI355_LD(float, wts, wts + t * top + k);
      if (x != nullptr && e >= num_real) {              // an identity expert: the input itself
        s += w * MI355_LDF(T, x, x + t * W + c);
        continue;
      }
      int64_t p = MI355_LD(int32_t, inv, inv + t * top + k);
      if (cap > 0) p += static_cast<int64_t>(e) * cap - MI355_LD(int32_t, offsets, offsets + e);   // y: every expert's rows padded to cap
      s += w * MI355_LDF(T, y, y + p * W + c);
    }
    if (shared != nullptr) s += sg * MI355_LDF(T, shared, shared + t * W + c);
    MI355_STF(T, out, out + t * W + c, s);
  }
}

}  // namespace mi355

using namespace mi355;

#define REQ_DTYPE(dtype) MI355_REQUIRE((dtype) >= MI355_BF16 && (dtype) <= MI355_F32, MI355_ERR_UNSUPPORTED, "dtype code %d", (dtype))

extern "C" int32_t mi355_moe_route(int32_t* ids, float* weights, const float* logits, int64_t logits_stride,
                                   const float* correction, int64_t num_tokens, int32_t experts, int32_t top,
                                   int32_t groups, int32_t keep, int32_t softmax, int32_t group_max, float weight_scale,
                                   void* stream) {
  MI355_REQUIRE(ids && weights && logits && correction, MI355_ERR_INVALID, "moe_route: null pointer");
  MI355_REQUIRE(logits_stride >= experts, MI355_ERR_INVALID, "moe_route: logit rows shorter than the experts");
  MI355_REQUIRE(num_tokens >= 0 && experts > 0 && top > 0 && groups > 0 && keep > 0 && keep <= groups &&
                    experts % groups == 0,
                MI355_ERR_INVALID, "moe_route: %d experts in %d groups, %d kept, %d chosen", experts, groups, keep, top);
  MI355_REQUIRE((top <= kMaxTop || experts <= 512) && groups <= kMaxGroups && top <= keep * (experts / groups),
                MI355_ERR_UNSUPPORTED,
                "moe_route: at most %d groups, %d chosen experts of more than 512; the kept groups must hold the %d chosen",
                kMaxGroups, kMaxTop, top);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 wgrid(static_cast<unsigned>((num_tokens + 3) / 4));
#define MI355_ROUTE(EPL)                                                                                            \
  hipLaunchKernelGGL((moe_route_wave_kernel<EPL>), wgrid, dim3(256), 0, s, ids, weights, logits, logits_stride,     \
                     correction, num_tokens, experts, top, groups, keep, softmax, group_max, weight_scale)
  if (experts <= 64) MI355_ROUTE(1);
  else if (experts <= 128) MI355_ROUTE(2);
  else if (experts <= 256) MI355_ROUTE(4);
  else if (experts <= 512) MI355_ROUTE(8);
  else                                                  // one thread per token
    hipLaunchKernelGGL(moe_route_kernel, dim3(static_cast<unsigned>((num_tokens + 63) / 64)), dim3(64), 0, s, ids, weights,
                       logits, logits_stride, correction, num_tokens, experts, top, groups, keep, softmax, group_max,
                       weight_scale);
#undef MI355_ROUTE
  return check_launch("moe_route");
}

extern "C" int32_t mi355_moe_sort(int32_t* offsets, int32_t* perm, int32_t* inv, const int32_t* ids, int64_t num_rows,
                                  int32_t experts, void* stream) {
  MI355_REQUIRE(offsets && perm && inv && ids, MI355_ERR_INVALID, "moe_sort: null pointer");
  MI355_REQUIRE(num_rows >= 0 && num_rows <= 0x7FFFFFFF && experts > 0 && experts <= 4096, MI355_ERR_INVALID,
                "moe_sort: sizes");
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), (2 * static_cast<size_t>(experts) + 1) * sizeof(int32_t),
                     static_cast<hipStream_t>(stream), offsets, perm, inv, ids, num_rows, experts);
  return check_launch("moe_sort");
}

extern "C" int32_t mi355_moe_gather_rows(void* xs, const void* x, const int32_t* perm, const int32_t* offsets,
                                         int32_t pad_to, int64_t num_rows, int32_t top, int32_t width, int32_t dtype,
                                         void* stream) {
  MI355_REQUIRE(xs && x && perm, MI355_ERR_INVALID, "moe_gather_rows: null pointer");
  MI355_REQUIRE(num_rows >= 0 && top > 0 && width > 0 && pad_to >= 0 && (pad_to == 0 || offsets != nullptr), MI355_ERR_INVALID,
                "moe_gather_rows: sizes");
  REQ_DTYPE(dtype);
  if (num_rows == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((moe_gather_rows_kernel<TT>), dim3(num_rows), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(xs), static_cast<const Elem<TT>::S*>(x), perm,
                                                  offsets, pad_to, top, width));
  return check_launch("moe_gather_rows");
}

extern "C" int32_t mi355_moe_gate_up_rows(void* act, const void* x, const void* w_gate_up, const int32_t* offsets,
                                          const int32_t* perm, int32_t experts, int32_t top, int32_t width, int32_t ff,
                                          int32_t act_fn, float limit, int32_t dtype, void* stream) {
  MI355_REQUIRE(act && x && w_gate_up && offsets && perm, MI355_ERR_INVALID, "moe_gate_up_rows: null pointer");
  MI355_REQUIRE(experts > 0 && experts <= 65535 && top > 0 && width > 0 && ff > 0, MI355_ERR_INVALID,
                "moe_gate_up_rows: sizes");
  REQ_DTYPE(dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>((ff + 3) / 4), static_cast<unsigned>(experts));
  if (dtype != MI355_F32 && width % 32 == 0 && ff % 16 == 0 && aligned16(x) && aligned16(w_gate_up) && aligned16(act)) {
    const dim3 mgrid(static_cast<unsigned>((ff / 16 + 3) / 4), static_cast<unsigned>(experts));
    if (dtype == MI355_BF16)
      hipLaunchKernelGGL((moe_gate_up_mfma_kernel<BF16>), mgrid, dim3(256), 0, s, static_cast<uint16_t*>(act),
                         static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w_gate_up), offsets, perm, top, width, ff,
                         act_fn, limit);
    else
      hipLaunchKernelGGL((moe_gate_up_mfma_kernel<F16>), mgrid, dim3(256), 0, s, static_cast<uint16_t*>(act),
                         static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w_gate_up), offsets, perm, top, width, ff,
                         act_fn, limit);
    return check_launch("moe_gate_up_rows (matrix cores)");
  }
  const bool vec = dtype != MI355_F32 && width % 8 == 0 && aligned16(x) && aligned16(w_gate_up);
  MI355_DISPATCH_DTYPE3(dtype, {
    if (vec)
      hipLaunchKernelGGL((moe_gate_up_rows_kernel<TT, true>), grid, dim3(256), 0, s, static_cast<Elem<TT>::S*>(act),
                         static_cast<const Elem<TT>::S*>(x), static_cast<const Elem<TT>::S*>(w_gate_up), offsets, perm, top,
                         width, ff, act_fn, limit);
    else
      hipLaunchKernelGGL((moe_gate_up_rows_kernel<TT, false>), grid, dim3(256), 0, s, static_cast<Elem<TT>::S*>(act),
                         static_cast<const Elem<TT>::S*>(x), static_cast<const Elem<TT>::S*>(w_gate_up), offsets, perm, top,
                         width, ff, act_fn, limit);
  });
  return check_launch("moe_gate_up_rows");
}

extern "C" int32_t mi355_moe_down_rows(void* y, const void* act, const void* w_down, const int32_t* offsets,
                                       int32_t experts, int32_t width, int32_t ff, int32_t dtype, void* stream) {
  MI355_REQUIRE(y && act && w_down && offsets, MI355_ERR_INVALID, "moe_down_rows: null pointer");
  MI355_REQUIRE(experts > 0 && experts <= 65535 && width > 0 && ff > 0, MI355_ERR_INVALID, "moe_down_rows: sizes");
  REQ_DTYPE(dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>((width + 3) / 4), static_cast<unsigned>(experts));
  if (dtype != MI355_F32 && ff % 32 == 0 && width % 16 == 0 && aligned16(act) && aligned16(w_down) && aligned16(y)) {
    const dim3 mgrid(static_cast<unsigned>((width / 16 + 3) / 4), static_cast<unsigned>(experts));
    if (dtype == MI355_BF16)
      hipLaunchKernelGGL((moe_down_mfma_kernel<BF16>), mgrid, dim3(256), 0, s, static_cast<uint16_t*>(y),
                         static_cast<const uint16_t*>(act), static_cast<const uint16_t*>(w_down), offsets, width, ff);
    else
      hipLaunchKernelGGL((moe_down_mfma_kernel<F16>), mgrid, dim3(256), 0, s, static_cast<uint16_t*>(y),
                         static_cast<const uint16_t*>(act), static_cast<const uint16_t*>(w_down), offsets, width, ff);
    return check_launch("moe_down_rows (matrix cores)");
  }
  const bool vec = dtype != MI355_F32 && ff % 8 == 0 && aligned16(act) && aligned16(w_down);
  MI355_DISPATCH_DTYPE3(dtype, {
    if (vec)
      hipLaunchKernelGGL((moe_down_rows_kernel<TT, true>), grid, dim3(256), 0, s, static_cast<Elem<TT>::S*>(y),
                         static_cast<const Elem<TT>::S*>(act), static_cast<const Elem<TT>::S*>(w_down), offsets, width, ff);
    else
      hipLaunchKernelGGL((moe_down_rows_kernel<TT, false>), grid, dim3(256), 0, s, static_cast<Elem<TT>::S*>(y),
                         static_cast<const Elem<TT>::S*>(act), static_cast<const Elem<TT>::S*>(w_down), offsets, width, ff);
  });
  return check_launch("moe_down_rows");
}

extern "C" int32_t mi355_moe_silu_and_mul(void* out, const void* x, int64_t num_rows, int32_t ff, int32_t act, float limit,
                                          int32_t dtype, void* stream) {
  MI355_REQUIRE(out && x, MI355_ERR_INVALID, "moe_silu_and_mul: null pointer");
  MI355_REQUIRE(num_rows >= 0 && ff > 0, MI355_ERR_INVALID, "moe_silu_and_mul: sizes");
  REQ_DTYPE(dtype);
  if (num_rows == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t blocks = (num_rows * ff + 255) / 256;
  const dim3 grid(static_cast<unsigned>(blocks > 65536 ? 65536 : blocks));
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((moe_silu_and_mul_kernel<TT>), grid, dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), static_cast<const Elem<TT>::S*>(x),
                                                  num_rows, ff, act, limit));
  return check_launch("moe_silu_and_mul");
}

extern "C" int32_t mi355_gated_act_rows(void* out, int64_t out_stride, const void* gate, const void* up, int64_t in_stride,
                                        int64_t num_rows, int32_t ff, int32_t act, float limit, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && gate && up, MI355_ERR_INVALID, "gated_act_rows: null pointer");
  MI355_REQUIRE(num_rows >= 0 && ff > 0 && out_stride >= ff && in_stride >= ff, MI355_ERR_INVALID, "gated_act_rows: sizes");
  REQ_DTYPE(dtype);
  if (num_rows == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype != MI355_F32 && ff % 8 == 0 && out_stride % 8 == 0 && in_stride % 8 == 0 && aligned16(out) && aligned16(gate) &&
      aligned16(up)) {
    const int64_t vb = (num_rows * (ff / 8) + 255) / 256;
    const dim3 vgrid(static_cast<unsigned>(vb > 65536 ? 65536 : vb));
    if (dtype == MI355_BF16)
      hipLaunchKernelGGL((gated_act_rows_vec_kernel<BF16>), vgrid, dim3(256), 0, s, static_cast<uint16_t*>(out), out_stride,
                         static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up), in_stride, num_rows, ff / 8, act,
                         limit);
    else
      hipLaunchKernelGGL((gated_act_rows_vec_kernel<F16>), vgrid, dim3(256), 0, s, static_cast<uint16_t*>(out), out_stride,
                         static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up), in_stride, num_rows, ff / 8, act,
                         limit);
    return check_launch("gated_act_rows");
  }
  const int64_t blocks = (num_rows * ff + 255) / 256;
  const dim3 grid(static_cast<unsigned>(blocks > 65536 ? 65536 : blocks));
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((gated_act_rows_kernel<TT>), grid, dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), out_stride,
                                                  static_cast<const Elem<TT>::S*>(gate), static_cast<const Elem<TT>::S*>(up),
                                                  in_stride, num_rows, ff, act, limit));
  return check_launch("gated_act_rows");
}

extern "C" int32_t mi355_moe_combine(void* out, const void* y, const int32_t* inv, const float* weights, const int32_t* ids,
                                     const int32_t* offsets, int32_t pad_to, int64_t num_tokens, int32_t top, int32_t width,
                                     const void* x, int32_t num_real, const void* shared, const float* shared_gate,
                                     int64_t shared_gate_stride, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && y && inv && weights, MI355_ERR_INVALID, "moe_combine: null pointer");
  MI355_REQUIRE(x == nullptr || (ids != nullptr && num_real >= 0), MI355_ERR_INVALID,
                "moe_combine: identity experts need the chosen ids");
  MI355_REQUIRE(num_tokens >= 0 && top > 0 && width > 0 && pad_to >= 0 && (pad_to == 0 || (ids && offsets)), MI355_ERR_INVALID,
                "moe_combine: sizes");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((moe_combine_kernel<TT>), dim3(num_tokens), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), static_cast<const Elem<TT>::S*>(y), inv,
                                                  weights, ids, offsets, pad_to, top, width,
                                                  static_cast<const Elem<TT>::S*>(x), num_real,
                                                  static_cast<const Elem<TT>::S*>(shared), shared_gate, shared_gate_stride));
  return check_launch("moe_combine");
}
