// Pointwise and normalisation kernels for decoders that keep the residual stream in fp32:
//   embed_scale_f32          resid = embed[id] * scale
//   embed_scale_pos_f32      resid = embed[id] * scale + pos_table[position]      (learned positions)
//   resid_add_f32            resid += other (fp32 rows) + rows (activation rows) + vec (one row, broadcast)
//   add_rms_norm_f32         resid += add; out = resid / rms(resid) * w      (w: one number or a vector)
//   rms_norm_mix_f32         resid += alpha * (xa / rms(xa) * wa + xb / rms(xb) * wb)
//   gelu_tanh_and_mul        out = gelu_tanh(gate) * up for rows holding gate | up
//   gated_head_rms_norm      out = o / rms(o) * w * act(gate) per (token, head) row of an fp32 tensor
//   softcap                  z = cap * tanh(z / cap)
//   group_rms_norm_f32       out = gn(x) * w: an RMS norm over each of `groups` equal consecutive parts of an
//                            fp32 row, to activation rows or (in place or not) to fp32 rows
//   gated_norm_resid_f32     resid += mult * gn(y * sigmoid(g + b)) * w: a sub-layer's result, gated element by
//                            element, normed in groups, scaled, added to the fp32 residual
//   rms_norm_rows            out = x / rms(x) * w for short rows that may be column slices (fp32 weight)
//   tanh_rows                out = tanh(x) for rows that may be column slices
// Every sum, mean and transcendental is fp32; activations are stored in bf16, fp16 or fp32
// (the dtype argument).  HBM-bound: one pass over the rows, one workgroup (or one wave) per row.
#include "common.h"

namespace mi355 {

template <typename T>
__global__ __launch_bounds__(256) void embed_scale_f32_kernel(float* __restrict__ out,
                                                              const typename Elem<T>::S* __restrict__ embed,
                                                              const int64_t* __restrict__ ids, int W, float scale) {
  const int64_t t = blockIdx.x;
  const int64_t id = MI355_LD(int64_t, ids, ids + t);
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    MI355_ST(float, out, out + t * W + c, MI355_LDF(T, embed, embed + id * W + c) * scale);
}

template <typename T>
__global__ __launch_bounds__(256) void embed_scale_pos_f32_kernel(float* __restrict__ out,
                                                                  const typename Elem<T>::S* __restrict__ embed,
                                                                  const typename Elem<T>::S* __restrict__ pos_table,
                                                                  const int64_t* __restrict__ ids,
                                                                  const int64_t* __restrict__ positions, int W,
                                                                  int64_t max_pos, float scale) {
  const int64_t t = blockIdx.x;
  const int64_t id = MI355_LD(int64_t, ids, ids + t);
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);     // (padding rows of a captured step: any row will do)
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    MI355_ST(float, out, out + t * W + c,
             MI355_LDF(T, embed, embed + id * W + c) * scale + MI355_LDF(T, pos_table, pos_table + p * W + c));
}

template <typename T>
__global__ __launch_bounds__(256) void resid_add_f32_kernel(float* __restrict__ resid, const float* __restrict__ other,
                                                            const typename Elem<T>::S* __restrict__ rows,
                                                            const typename Elem<T>::S* __restrict__ vec, int W) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = MI355_LD(float, resid, resid + t * W + c);
    if (other != nullptr) v += MI355_LD(float, other, other + t * W + c);
    if (rows != nullptr) v += MI355_LDF(T, rows, rows + t * W + c);
    if (vec != nullptr) v += MI355_LDF(T, vec, vec + c);
    MI355_ST(float, resid, resid + t * W + c, v);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void add_rms_norm_f32_kernel(typename Elem<T>::S* __restrict__ out,
                                                               float* __restrict__ resid,
                                                               const typename Elem<T>::S* __restrict__ add,
                                                               const typename Elem<T>::S* __restrict__ weight,
                                                               int weight_numel, int W, float eps) {
  __shared__ float scratch[32];
  const int64_t t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = MI355_LD(float, resid, resid + t * W + c);
    if (add != nullptr) {
      v += MI355_LDF(T, add, add + t * W + c);
      MI355_ST(float, resid, resid + t * W + c, v);
    }
    ss += v * v;
  }
  ss = block_sum32(ss, scratch);
  const float r = 1.0f / sqrtf(ss / static_cast<float>(W) + eps);
  const float g1 = weight_numel == 1 ? MI355_LDF(T, weight, weight) : 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = MI355_LD(float, resid, resid + t * W + c);      // own writes of this thread: same c
    const float g = weight_numel == 1 ? g1 : MI355_LDF(T, weight, weight + c);
    MI355_STF(T, out, out + t * W + c, v * r * g);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rms_norm_mix_f32_kernel(float* __restrict__ resid,
                                                               const typename Elem<T>::S* __restrict__ xa,
                                                               const typename Elem<T>::S* __restrict__ wa,
                                                               const typename Elem<T>::S* __restrict__ xb,
                                                               const typename Elem<T>::S* __restrict__ wb, int W,
                                                               float eps, float alpha) {
  __shared__ float scratch[32];
  const int64_t t = blockIdx.x;
  float sa = 0.f, sb = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float a = MI355_LDF(T, xa, xa + t * W + c);
    sa += a * a;
    if (xb != nullptr) {
      const float b = MI355_LDF(T, xb, xb + t * W + c);
      sb += b * b;
    }
  }
  sa = block_sum32(sa, scratch);
  sb = block_sum32(sb, scratch);
  const float ra = 1.0f / sqrtf(sa / static_cast<float>(W) + eps);
  const float rb = 1.0f / sqrtf(sb / static_cast<float>(W) + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float m = MI355_LDF(T, xa, xa + t * W + c) * ra * MI355_LDF(T, wa, wa + c);
    if (xb != nullptr) m += MI355_LDF(T, xb, xb + t * W + c) * rb * MI355_LDF(T, wb, wb + c);
    const float v = MI355_LD(float, resid, resid + t * W + c);
    MI355_ST(float, resid, resid + t * W + c, v + alpha * m);
  }
}

// 0.5 z (1 + tanh(w)) = z / (1 + exp(-2 w)), w = sqrt(2 / pi) (z + 0.044715 z^3)
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return z / (1.0f + expf(-1.5957691216057308f * (z + 0.044715f * z * z * z)));
}

// 16-bit rows, 8 elements per thread (16-byte loads and stores)
template <typename T>
__global__ __launch_bounds__(256) void gelu_tanh_and_mul_vec_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ x,
                                                                    int64_t x_stride, int64_t num_tokens, int inter) {
  const int vec_per_row = inter >> 3;
  const int64_t total = num_tokens * vec_per_row;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t row = i / vec_per_row;
    const int v = static_cast<int>(i % vec_per_row);
    const uint16_t* xr = x + row * x_stride;
    float g[8], u[8], y[8];
    unpack8<T>(MI355_LD(uint4, x, xr + 8 * v), g);
    unpack8<T>(MI355_LD(uint4, x, xr + inter + 8 * v), u);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      y[j] = g[j] * __frcp_rn(1.0f + __expf(-1.5957691216057308f * (g[j] + 0.044715f * g[j] * g[j] * g[j]))) * u[j];
    MI355_ST(uint4, out, out + row * inter + 8 * v, pack8<T>(y));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_tanh_and_mul_kernel(typename Elem<T>::S* __restrict__ out,
                                                                const typename Elem<T>::S* __restrict__ x,
                                                                int64_t x_stride, int64_t num_tokens, int inter) {
  const int64_t total = num_tokens * inter;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t row = i / inter;
    const int c = static_cast<int>(i % inter);
    const float g = MI355_LDF(T, x, x + row * x_stride + c);
    const float u = MI355_LDF(T, x, x + row * x_stride + inter + c);
    MI355_STF(T, out, out + row * inter + c, gelu_tanh_f(g) * u);
  }
}

// one wave per (token, head) row of o [rows = T * H][dv]
template <typename T>
__global__ __launch_bounds__(256) void gated_head_rms_norm_kernel(typename Elem<T>::S* __restrict__ out,
                                                                  const float* __restrict__ o,
                                                                  const typename Elem<T>::S* __restrict__ gate,
                                                                  int64_t gate_stride, const float* __restrict__ w,
                                                                  int w_heads, int64_t rows, int H, int dv, float eps,
                                                                  int act) {
  const int64_t row = blockIdx.x * static_cast<int64_t>(blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = row / H;
  const int h = static_cast<int>(row % H);
  float ss = 0.f;
  for (int c = lane; c < dv; c += 64) {
    const float v = MI355_LD(float, o, o + row * dv + c);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / static_cast<float>(dv) + eps);
  for (int c = lane; c < dv; c += 64) {
    const float v = MI355_LD(float, o, o + row * dv + c);
    const float g = MI355_LDF(T, gate, gate + t * gate_stride + static_cast<int64_t>(h) * dv + c);
    const float s = 1.0f / (1.0f + expf(-g));
    const float a = act == 0 ? g * s : s;
    MI355_STF(T, out, out + row * dv + c, v * r * MI355_LD(float, w, w + (w_heads > 1 ? h * dv : 0) + c) * a);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softcap_kernel(typename Elem<T>::S* __restrict__ z, int64_t n, float cap) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    MI355_STF(T, z, z + i, cap * tanhf(MI355_LDF(T, z, z + i) / cap));
}

constexpr int kMaxNormGroups = 64;

// rg[g] = 1 / sqrt(mean of sq(c) over the columns c of group g + eps), for every group of gw columns
template <typename F>
__device__ __forceinline__ void group_rsqrt(F sq, int groups, int gw, float eps, float* rg, float* scratch) {
  for (int g = 0; g < groups; ++g) {
    float s = 0.f;
    for (int c = g * gw + threadIdx.x; c < (g + 1) * gw; c += blockDim.x) s += sq(c);
    s = block_sum32(s, scratch);
    if (threadIdx.x == 0) rg[g] = 1.0f / sqrtf(s / static_cast<float>(gw) + eps);
  }
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(256) void group_rms_norm_f32_kernel(typename Elem<T>::S* __restrict__ out,
                                                                 float* out_f32, const float* x,   // may be one buffer
                                                                 const float* __restrict__ weight, int W, int groups,
                                                                 float eps) {
  __shared__ float scratch[32];
  __shared__ float rg[kMaxNormGroups];
  const int64_t t = blockIdx.x;
  const int gw = W / groups;
  group_rsqrt([&](int c) { const float v = MI355_LD(float, x, x + t * W + c); return v * v; }, groups, gw, eps, rg, scratch);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = MI355_LD(float, x, x + t * W + c) * rg[c / gw] * MI355_LD(float, weight, weight + c);
    if (out_f32 != nullptr) MI355_ST(float, out_f32, out_f32 + t * W + c, v);
    else MI355_STF(T, out, out + t * W + c, v);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_norm_resid_f32_kernel(float* __restrict__ resid,
                                                                   const typename Elem<T>::S* __restrict__ y,
                                                                   const typename Elem<T>::S* __restrict__ gate,
                                                                   int64_t gate_stride, const float* __restrict__ bias,
                                                                   const float* __restrict__ weight, int W, int groups,
                                                                   float eps, float mult) {
  __shared__ float scratch[32];
  __shared__ float rg[kMaxNormGroups];
  const int64_t t = blockIdx.x;
  const int gw = W / groups;
  auto gated = [&](int c) {
    const float z = MI355_LDF(T, gate, gate + t * gate_stride + c) + MI355_LD(float, bias, bias + c);
    return MI355_LDF(T, y, y + t * W + c) / (1.0f + expf(-z));
  };
  group_rsqrt([&](int c) { const float v = gated(c); return v * v; }, groups, gw, eps, rg, scratch);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = gated(c) * rg[c / gw] * MI355_LD(float, weight, weight + c);
    MI355_ST(float, resid, resid + t * W + c, MI355_LD(float, resid, resid + t * W + c) + mult * v);
  }
}

// one wave per row
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_rows_kernel(typename Elem<T>::S* __restrict__ out,
                                                            const typename Elem<T>::S* __restrict__ x, int64_t x_stride,
                                                            const float* __restrict__ weight, int64_t rows, int n,
                                                            float eps) {
  const int64_t row = blockIdx.x * static_cast<int64_t>(blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  float ss = 0.f;
  for (int c = lane; c < n; c += 64) {
    const float v = MI355_LDF(T, x, x + row * x_stride + c);
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(n) + eps);
  for (int c = lane; c < n; c += 64)
    MI355_STF(T, out, out + row * n + c, MI355_LDF(T, x, x + row * x_stride + c) * r * MI355_LD(float, weight, weight + c));
}

template <typename T>
__global__ __launch_bounds__(256) void tanh_rows_kernel(typename Elem<T>::S* __restrict__ out,
                                                        const typename Elem<T>::S* __restrict__ x, int64_t x_stride,
                                                        int64_t rows, int n) {
  const int64_t total = rows * n;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    MI355_STF(T, out, out + i, tanhf(MI355_LDF(T, x, x + (i / n) * x_stride + i % n)));
}

// out[t] = embed[id] + bigram[row] + sinusoid(position), float32 rows.  row = (previous token * mul_prev
// + id * mul_cur) mod buckets, `buckets` itself for a sequence's first token; the previous token of a
// chunk's first row is the sequence's state (prev_tokens[slot], written by prev_token_update after
// this launch).  Entry 2i of the sinusoid is sin(p * freq[i]), entry 2i + 1 the cosine; angles in fp32.
template <typename T>
__global__ __launch_bounds__(256) void embed_bigram_pos_f32_kernel(
    float* __restrict__ out, const typename Elem<T>::S* __restrict__ embed, const typename Elem<T>::S* __restrict__ bigram,
    const int64_t* __restrict__ ids, const int64_t* __restrict__ positions, const int32_t* __restrict__ cu_seqlens,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ state_slots, const int32_t* __restrict__ prev_tokens,
    const float* __restrict__ freq, int W, int64_t vocab, int64_t buckets, int64_t mul_prev, int64_t mul_cur) {
  const int64_t t = blockIdx.x;
  int64_t id = MI355_LD(int64_t, ids, ids + t);
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const int64_t p = MI355_LD(int64_t, positions, positions + t);
  const typename Elem<T>::S* brow = nullptr;
  if (bigram != nullptr) {
    int64_t row = buckets;
    if (p > 0) {
      const int seq = MI355_LD(int32_t, tok_seq, tok_seq + t);
      int64_t prev = t == MI355_LD(int32_t, cu_seqlens, cu_seqlens + seq)
                         ? MI355_LD(int32_t, prev_tokens, prev_tokens + MI355_LD(int32_t, state_slots, state_slots + seq))
                         : MI355_LD(int64_t, ids, ids + t - 1);
      prev = prev < 0 ? 0 : (prev >= vocab ? vocab - 1 : prev);
      row = (prev * mul_prev + id * mul_cur) % buckets;
    }
    brow = bigram + row * W;
  }
  const float pf = static_cast<float>(p);
  for (int i = threadIdx.x; 2 * i < W; i += blockDim.x) {     // a pair of columns shares its angle
    float sn = 0.f, cs = 0.f;
    if (freq != nullptr) sincosf(pf * MI355_LD(float, freq, freq + i), &sn, &cs);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = 2 * i + j;
      if (c >= W) break;
      float v = MI355_LDF(T, embed, embed + id * W + c);
      if (brow != nullptr) v += MI355_LDF(T, bigram, brow + c);
      MI355_ST(float, out, out + t * W + c, v + (j ? cs : sn));
    }
  }
}

// prev_tokens[slot of chunk s] = the chunk's last token
__global__ __launch_bounds__(256) void prev_token_update_kernel(int32_t* __restrict__ prev_tokens,
                                                                const int64_t* __restrict__ ids,
                                                                const int32_t* __restrict__ cu_seqlens,
                                                                const int32_t* __restrict__ state_slots, int S) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= S) return;
  const int end = MI355_LD(int32_t, cu_seqlens, cu_seqlens + s + 1);
  if (end <= MI355_LD(int32_t, cu_seqlens, cu_seqlens + s)) return;
  MI355_ST(int32_t, prev_tokens, prev_tokens + MI355_LD(int32_t, state_slots, state_slots + s),
           static_cast<int32_t>(MI355_LD(int64_t, ids, ids + end - 1)));
}

// out = relu(x)^2
template <typename T>
__global__ __launch_bounds__(256) void relu_squared_kernel(typename Elem<T>::S* __restrict__ out,
                                                           const typename Elem<T>::S* __restrict__ x, int64_t n) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const float v = fmaxf(MI355_LDF(T, x, x + i), 0.f);
    MI355_STF(T, out, out + i, v * v);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void relu_squared_vec_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ x,
                                                               int64_t nvec) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < nvec;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    float f[8];
    unpack8<T>(MI355_LD(uint4, x, x + 8 * i), f);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = fmaxf(f[j], 0.f);
      f[j] = v * v;
    }
    MI355_ST(uint4, out, out + 8 * i, pack8<T>(f));
  }
}

static inline dim3 stride_grid(int64_t total) {
  const int64_t blocks = (total + 255) / 256;
  return dim3(static_cast<unsigned>(blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks)));
}

}  // namespace mi355

using namespace mi355;

#define REQ_DTYPE(dtype) MI355_REQUIRE((dtype) >= MI355_BF16 && (dtype) <= MI355_F32, MI355_ERR_UNSUPPORTED, "dtype code %d", (dtype))

extern "C" int32_t mi355_embed_scale_f32(float* out, const void* embed, const int64_t* ids, int64_t num_tokens,
                                         int32_t width, int64_t vocab, float scale, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && embed && ids, MI355_ERR_INVALID, "embed_scale_f32: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && width > 0 && vocab > 0, MI355_ERR_INVALID, "embed_scale_f32: sizes");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((embed_scale_f32_kernel<TT>), dim3(num_tokens), dim3(256), 0, s, out,
                                                  static_cast<const Elem<TT>::S*>(embed), ids, width, scale));
  return check_launch("embed_scale_f32");
}

extern "C" int32_t mi355_embed_scale_pos_f32(float* out, const void* embed, const void* pos_table, const int64_t* ids,
                                             const int64_t* positions, int64_t num_tokens, int32_t width, int64_t vocab,
                                             int64_t max_pos, float scale, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && embed && pos_table && ids && positions, MI355_ERR_INVALID, "embed_scale_pos_f32: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && width > 0 && vocab > 0 && max_pos > 0, MI355_ERR_INVALID, "embed_scale_pos_f32: sizes");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((embed_scale_pos_f32_kernel<TT>), dim3(num_tokens), dim3(256), 0, s, out,
                                                  static_cast<const Elem<TT>::S*>(embed),
                                                  static_cast<const Elem<TT>::S*>(pos_table), ids, positions, width,
                                                  max_pos, scale));
  return check_launch("embed_scale_pos_f32");
}

extern "C" int32_t mi355_embed_bigram_pos_f32(float* out, const void* embed, const void* bigram, const int64_t* ids,
                                              const int64_t* positions, const int32_t* cu_seqlens, const int32_t* tok_seq,
                                              const int32_t* state_slots, const int32_t* prev_tokens, const float* freq,
                                              int64_t num_tokens, int32_t width, int64_t vocab, int64_t buckets,
                                              int64_t mul_prev, int64_t mul_cur, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && embed && ids && positions, MI355_ERR_INVALID, "embed_bigram_pos_f32: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && width > 0 && vocab > 0, MI355_ERR_INVALID, "embed_bigram_pos_f32: sizes");
  MI355_REQUIRE(bigram == nullptr || (cu_seqlens && tok_seq && state_slots && prev_tokens && buckets > 0 && mul_prev >= 0 &&
                                      mul_cur >= 0 && vocab <= (1ll << 31) && mul_prev < (1ll << 31) && mul_cur < (1ll << 31)),
                MI355_ERR_INVALID, "embed_bigram_pos_f32: a bigram table needs the chunk layout, the state and its constants");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((embed_bigram_pos_f32_kernel<TT>), dim3(num_tokens), dim3(256), 0, s, out,
                                                  static_cast<const Elem<TT>::S*>(embed),
                                                  static_cast<const Elem<TT>::S*>(bigram), ids, positions, cu_seqlens,
                                                  tok_seq, state_slots, prev_tokens, freq, width, vocab, buckets, mul_prev,
                                                  mul_cur));
  return check_launch("embed_bigram_pos_f32");
}

extern "C" int32_t mi355_prev_token_update(int32_t* prev_tokens, const int64_t* ids, const int32_t* cu_seqlens,
                                           const int32_t* state_slots, int32_t num_seqs, void* stream) {
  MI355_REQUIRE(prev_tokens && ids && cu_seqlens && state_slots, MI355_ERR_INVALID, "prev_token_update: null pointer");
  MI355_REQUIRE(num_seqs >= 0, MI355_ERR_INVALID, "prev_token_update: sizes");
  if (num_seqs == 0) return MI355_OK;
  hipLaunchKernelGGL(prev_token_update_kernel, dim3((num_seqs + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                     prev_tokens, ids, cu_seqlens, state_slots, num_seqs);
  return check_launch("prev_token_update");
}

extern "C" int32_t mi355_relu_squared(void* out, const void* x, int64_t numel, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && x, MI355_ERR_INVALID, "relu_squared: null pointer");
  MI355_REQUIRE(numel >= 0, MI355_ERR_INVALID, "relu_squared: sizes");
  REQ_DTYPE(dtype);
  if (numel == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype != MI355_F32 && numel % 8 == 0 && aligned16(out) && aligned16(x)) {
    if (dtype == MI355_BF16)
      hipLaunchKernelGGL((relu_squared_vec_kernel<BF16>), stride_grid(numel / 8), dim3(256), 0, s,
                         static_cast<uint16_t*>(out), static_cast<const uint16_t*>(x), numel / 8);
    else
      hipLaunchKernelGGL((relu_squared_vec_kernel<F16>), stride_grid(numel / 8), dim3(256), 0, s,
                         static_cast<uint16_t*>(out), static_cast<const uint16_t*>(x), numel / 8);
    return check_launch("relu_squared");
  }
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((relu_squared_kernel<TT>), stride_grid(numel), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), static_cast<const Elem<TT>::S*>(x), numel));
  return check_launch("relu_squared");
}

extern "C" int32_t mi355_resid_add_f32(float* resid, const float* other, const void* rows, const void* vec, int64_t num_tokens,
                                       int32_t width, int32_t dtype, void* stream) {
  MI355_REQUIRE(resid, MI355_ERR_INVALID, "resid_add_f32: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && width > 0, MI355_ERR_INVALID, "resid_add_f32: sizes");
  REQ_DTYPE(dtype);
  if (num_tokens == 0 || (!other && !rows && !vec)) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((resid_add_f32_kernel<TT>), dim3(num_tokens), dim3(256), 0, s, resid,
                                                  other, static_cast<const Elem<TT>::S*>(rows),
                                                  static_cast<const Elem<TT>::S*>(vec), width));
  return check_launch("resid_add_f32");
}

extern "C" int32_t mi355_add_rms_norm_f32(void* out, float* resid, const void* add, const void* weight,
                                          int32_t weight_numel, int64_t num_tokens, int32_t width, float eps,
                                          int32_t dtype, void* stream) {
  MI355_REQUIRE(out && resid && weight, MI355_ERR_INVALID, "add_rms_norm_f32: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && width > 0, MI355_ERR_INVALID, "add_rms_norm_f32: sizes");
  MI355_REQUIRE(weight_numel == 1 || weight_numel == width, MI355_ERR_INVALID,
                "add_rms_norm_f32: the weight is one number or one per column (%d for width %d)", weight_numel, width);
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((add_rms_norm_f32_kernel<TT>), dim3(num_tokens), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), resid,
                                                  static_cast<const Elem<TT>::S*>(add),
                                                  static_cast<const Elem<TT>::S*>(weight), weight_numel, width, eps));
  return check_launch("add_rms_norm_f32");
}

extern "C" int32_t mi355_rms_norm_mix_f32(float* resid, const void* xa, const void* wa, const void* xb, const void* wb,
                                          int64_t num_tokens, int32_t width, float eps, float alpha, int32_t dtype,
                                          void* stream) {
  MI355_REQUIRE(resid && xa && wa && ((xb == nullptr) == (wb == nullptr)), MI355_ERR_INVALID,
                "rms_norm_mix_f32: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && width > 0, MI355_ERR_INVALID, "rms_norm_mix_f32: sizes");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((rms_norm_mix_f32_kernel<TT>), dim3(num_tokens), dim3(256), 0, s, resid,
                                                  static_cast<const Elem<TT>::S*>(xa), static_cast<const Elem<TT>::S*>(wa),
                                                  static_cast<const Elem<TT>::S*>(xb), static_cast<const Elem<TT>::S*>(wb),
                                                  width, eps, alpha));
  return check_launch("rms_norm_mix_f32");
}

extern "C" int32_t mi355_gelu_tanh_and_mul(void* out, const void* x, int64_t x_stride, int64_t num_tokens,
                                           int32_t inter, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && x, MI355_ERR_INVALID, "gelu_tanh_and_mul: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && inter > 0 && x_stride >= 2 * static_cast<int64_t>(inter), MI355_ERR_INVALID,
                "gelu_tanh_and_mul: sizes");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype != MI355_F32 && inter % 8 == 0 && x_stride % 8 == 0 && aligned16(x) && aligned16(out)) {
    const dim3 grid = stride_grid(num_tokens * (inter / 8));
    if (dtype == MI355_BF16)
      hipLaunchKernelGGL((gelu_tanh_and_mul_vec_kernel<BF16>), grid, dim3(256), 0, s, static_cast<uint16_t*>(out),
                         static_cast<const uint16_t*>(x), x_stride, num_tokens, inter);
    else
      hipLaunchKernelGGL((gelu_tanh_and_mul_vec_kernel<F16>), grid, dim3(256), 0, s, static_cast<uint16_t*>(out),
                         static_cast<const uint16_t*>(x), x_stride, num_tokens, inter);
    return check_launch("gelu_tanh_and_mul");
  }
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((gelu_tanh_and_mul_kernel<TT>), stride_grid(num_tokens * inter), dim3(256),
                                                  0, s, static_cast<Elem<TT>::S*>(out),
                                                  static_cast<const Elem<TT>::S*>(x), x_stride, num_tokens, inter));
  return check_launch("gelu_tanh_and_mul");
}

extern "C" int32_t mi355_gated_head_rms_norm(void* out, const float* o, const void* gate, int64_t gate_stride,
                                             const float* weight, int32_t weight_heads, int64_t num_tokens,
                                             int32_t num_heads, int32_t head_dim, float eps, int32_t activation,
                                             int32_t dtype, void* stream) {
  MI355_REQUIRE(out && o && gate && weight, MI355_ERR_INVALID, "gated_head_rms_norm: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && head_dim > 0 &&
                    gate_stride >= static_cast<int64_t>(num_heads) * head_dim,
                MI355_ERR_INVALID, "gated_head_rms_norm: sizes");
  MI355_REQUIRE(activation == 0 || activation == 1, MI355_ERR_INVALID,
                "gated_head_rms_norm: activation is 0 (silu) or 1 (sigmoid)");
  MI355_REQUIRE(weight_heads == 1 || weight_heads == num_heads, MI355_ERR_INVALID,
                "gated_head_rms_norm: the weight is one head's (1) or all heads' (%d), not %d", num_heads, weight_heads);
  REQ_DTYPE(dtype);
  const int64_t rows = num_tokens * num_heads;
  if (rows == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((gated_head_rms_norm_kernel<TT>), dim3((rows + 3) / 4), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), o,
                                                  static_cast<const Elem<TT>::S*>(gate), gate_stride, weight,
                                                  weight_heads, rows, num_heads, head_dim, eps, activation));
  return check_launch("gated_head_rms_norm");
}

extern "C" int32_t mi355_softcap(void* z, int64_t numel, float cap, int32_t dtype, void* stream) {
  MI355_REQUIRE(z, MI355_ERR_INVALID, "softcap: null pointer");
  MI355_REQUIRE(numel >= 0 && cap > 0.f, MI355_ERR_INVALID, "softcap: sizes");
  REQ_DTYPE(dtype);
  if (numel == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((softcap_kernel<TT>), stride_grid(numel), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(z), numel, cap));
  return check_launch("softcap");
}

extern "C" int32_t mi355_group_rms_norm_f32(void* out, float* out_f32, const float* x, const float* weight,
                                            int64_t num_tokens, int32_t width, int32_t groups, float eps, int32_t dtype,
                                            void* stream) {
  MI355_REQUIRE((out != nullptr) != (out_f32 != nullptr) && x && weight, MI355_ERR_INVALID,
                "group_rms_norm_f32: null pointer, or both outputs given");
  MI355_REQUIRE(num_tokens >= 0 && width > 0 && groups > 0 && groups <= kMaxNormGroups && width % groups == 0,
                MI355_ERR_INVALID, "group_rms_norm_f32: width %d in %d groups (at most %d)", width, groups, kMaxNormGroups);
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((group_rms_norm_f32_kernel<TT>), dim3(num_tokens), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), out_f32, x, weight, width, groups, eps));
  return check_launch("group_rms_norm_f32");
}

extern "C" int32_t mi355_gated_norm_resid_f32(float* resid, const void* y, const void* gate, int64_t gate_stride,
                                              const float* bias, const float* weight, int64_t num_tokens, int32_t width,
                                              int32_t groups, float eps, float mult, int32_t dtype, void* stream) {
  MI355_REQUIRE(resid && y && gate && bias && weight, MI355_ERR_INVALID, "gated_norm_resid_f32: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && width > 0 && groups > 0 && groups <= kMaxNormGroups && width % groups == 0 &&
                    gate_stride >= width,
                MI355_ERR_INVALID, "gated_norm_resid_f32: width %d in %d groups (at most %d)", width, groups,
                kMaxNormGroups);
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((gated_norm_resid_f32_kernel<TT>), dim3(num_tokens), dim3(256), 0, s,
                                                  resid, static_cast<const Elem<TT>::S*>(y),
                                                  static_cast<const Elem<TT>::S*>(gate), gate_stride, bias, weight, width,
                                                  groups, eps, mult));
  return check_launch("gated_norm_resid_f32");
}

extern "C" int32_t mi355_rms_norm_rows(void* out, const void* x, int64_t x_stride, const float* weight, int64_t num_rows,
                                       int32_t n, float eps, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && x && weight, MI355_ERR_INVALID, "rms_norm_rows: null pointer");
  MI355_REQUIRE(num_rows >= 0 && n > 0 && x_stride >= n, MI355_ERR_INVALID, "rms_norm_rows: sizes");
  REQ_DTYPE(dtype);
  if (num_rows == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((rms_norm_rows_kernel<TT>), dim3((num_rows + 3) / 4), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), static_cast<const Elem<TT>::S*>(x),
                                                  x_stride, weight, num_rows, n, eps));
  return check_launch("rms_norm_rows");
}

extern "C" int32_t mi355_tanh_rows(void* out, const void* x, int64_t x_stride, int64_t num_rows, int32_t n, int32_t dtype,
                                   void* stream) {
  MI355_REQUIRE(out && x, MI355_ERR_INVALID, "tanh_rows: null pointer");
  MI355_REQUIRE(num_rows >= 0 && n > 0 && x_stride >= n, MI355_ERR_INVALID, "tanh_rows: sizes");
  REQ_DTYPE(dtype);
  if (num_rows == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((tanh_rows_kernel<TT>), stride_grid(num_rows * n), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(out), static_cast<const Elem<TT>::S*>(x),
                                                  x_stride, num_rows, n));
  return check_launch("tanh_rows");
}
