// Softmax attention inside blocks of positions with a logarithmic distance penalty, over the engine's
// paged K/V, and the kernel that prepares its operands.  Packed batches as in seqmix.hip: chunks
// (whole prompts, portions, single decoded tokens) side by side, tok_seq / positions per row.
//
//   qk_norm_kv_write      q <- rms(q) * wq per head, in place; K pages <- rms(k) * wk per head; V pages <- v
//                         (any rows of the caller's choice: a design whose values are its unnormed keys
//                         passes k again)
//   softmax_bias_attn     out[t,h] = gate[t,h,:] * sum_j softmax_j(q.k_j * scale - r1[h] ln(1 + r2[h] (p - j))) v_j
//                         over the keys j <= p of p's block: lo = (p / block) * block (block 0: lo = 0), and
//                         with a window also j > p - window.  Blocks are counted from position 0 of the
//                         sequence.  gate: sigmoid of one number per head or per output channel.
//                         sink (fp32, one score per head, may be null): the softmax denominator holds one
//                         more term exp(sink[h]) that carries no value.  Output rows are out_stride apart
//                         (a column slice of a wider buffer is fine).
// Norms, scores, penalties, softmax and accumulators are fp32; pages and activations are stored in
// the dtype argument's type.  K pages [blocks, kv_heads, 16, dim], V pages [blocks, kv_heads, vdim, 16].
#include "common.h"

namespace mi355 {

constexpr int kPageB = MI355_BLOCK_SIZE;
constexpr float kLog2eB = 1.4426950408889634f;
constexpr float kLazyLog2 = 8.0f;

// one workgroup per packed row, one wave per head in turn
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_kv_write_kernel(
    typename Elem<T>::S* __restrict__ q, int64_t q_stride, const typename Elem<T>::S* __restrict__ k, int64_t k_stride,
    const typename Elem<T>::S* __restrict__ v, int64_t v_stride, const float* __restrict__ wq, const float* __restrict__ wk,
    const int64_t* __restrict__ slot_mapping, typename Elem<T>::S* __restrict__ k_cache,
    typename Elem<T>::S* __restrict__ v_cache, int H, int G, int d, int dv, float eps) {
  typedef typename Elem<T>::S E;
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const int64_t slot = MI355_LD(int64_t, slot_mapping, slot_mapping + t);
  const int64_t page = slot / kPageB, off = slot % kPageB;
  for (int h = wave; h < H + G; h += nw) {
    const bool is_q = h < H;
    const int g = h - H;
    if (!is_q && slot < 0) continue;
    const E* src = is_q ? q + t * q_stride + static_cast<int64_t>(h) * d : k + t * k_stride + static_cast<int64_t>(g) * d;
    [[maybe_unused]] const void* base = is_q ? static_cast<const void*>(q) : static_cast<const void*>(k);
    float ss = 0.f;
    for (int i = lane; i < d; i += 64) {
      const float x = MI355_LDF(T, base, src + i);
      ss += x * x;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
    const float* w = is_q ? wq : wk;
    for (int i = lane; i < d; i += 64) {
      const float x = MI355_LDF(T, base, src + i) * r * MI355_LD(float, w, w + i);
      if (is_q) MI355_STF(T, q, q + t * q_stride + static_cast<int64_t>(h) * d + i, x);
      else MI355_STF(T, k_cache, k_cache + ((page * G + g) * kPageB + off) * d + i, x);
    }
  }
  if (slot < 0) return;
  for (int i = threadIdx.x; i < G * dv; i += blockDim.x) {
    const int g = i / dv, j = i % dv;
    MI355_ST(E, v_cache, v_cache + ((page * G + g) * dv + j) * kPageB + off,
             MI355_LD(E, v, v + t * v_stride + static_cast<int64_t>(g) * dv + j));
  }
}

__device__ __forceinline__ int64_t first_visible(int64_t p, int block, int window) {
  int64_t lo = block > 0 ? (p / block) * block : 0;
  if (window > 0 && p - window + 1 > lo) lo = p - window + 1;
  return lo;
}

// One wave per (packed row, query head): 64 keys at a time, a key's score per lane, running maximum
// and sum, then every lane accumulates its value channels over the 64 keys.  Any storage type and
// any head size; serves portions of prompts and decoded tokens alike.
template <typename T, int DV_PER_LANE>
__global__ __launch_bounds__(64) void softmax_bias_attn_kernel(
    typename Elem<T>::S* __restrict__ out, const typename Elem<T>::S* __restrict__ q, int64_t q_stride,
    const typename Elem<T>::S* __restrict__ k_cache, const typename Elem<T>::S* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ tok_seq,
    const int64_t* __restrict__ positions, const float* __restrict__ r1, const float* __restrict__ r2,
    const typename Elem<T>::S* __restrict__ gate, int64_t gate_stride, int gate_per_channel, int H, int G, int d, int dv,
    int block, int window, float scale, const float* __restrict__ sink, int64_t out_stride) {
  extern __shared__ float lds[];                        // q [d] | w [64]
  float* qs = lds;
  float* ws = lds + d;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, g = h / (H / G), lane = threadIdx.x;
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  if (p < 0) p = 0;
  if (p >= static_cast<int64_t>(max_blocks) * kPageB) p = static_cast<int64_t>(max_blocks) * kPageB - 1;   // never past the table
  const int32_t* bt = block_tables + static_cast<int64_t>(MI355_LD(int32_t, tok_seq, tok_seq + t)) * max_blocks;
  for (int i = lane; i < d; i += 64) qs[i] = MI355_LDF(T, q, q + t * q_stride + static_cast<int64_t>(h) * d + i);
  const float a1 = r1 != nullptr ? MI355_LD(float, r1, r1 + h) : 0.f;
  const float a2 = r2 != nullptr ? MI355_LD(float, r2, r2 + h) : 0.f;
  float acc[DV_PER_LANE];
#pragma unroll
  for (int i = 0; i < DV_PER_LANE; ++i) acc[i] = 0.f;
  float m = -__builtin_inff(), l = 0.f;
  const int64_t lo = first_visible(p, block, window);
  __syncthreads();
  for (int64_t base = lo; base <= p; base += 64) {
    const int64_t j = base + lane;
    float s = -__builtin_inff();
    if (j <= p) {
      const int64_t page = MI355_LD(int32_t, block_tables, bt + j / kPageB);
      const typename Elem<T>::S* kr = k_cache + ((page * G + g) * kPageB + j % kPageB) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot += qs[i] * MI355_LDF(T, k_cache, kr + i);
      s = dot * scale - a1 * log1pf(a2 * static_cast<float>(p - j));
    }
    float tm = s;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) tm = fmaxf(tm, __shfl_xor(tm, o, 64));
    const float mn = fmaxf(m, tm);                      // (finite: the tile's first key is visible)
    const float corr = expf(m - mn);
    const float w = j <= p ? expf(s - mn) : 0.f;
    l = l * corr + wave_sum(w);
    m = mn;
    ws[lane] = w;
    __syncthreads();
    const int n = static_cast<int>((p - base + 1) < 64 ? (p - base + 1) : 64);
#pragma unroll
    for (int i = 0; i < DV_PER_LANE; ++i) acc[i] *= corr;
    for (int jj = 0; jj < n; ++jj) {
      const int64_t key = base + jj;
      const int64_t page = MI355_LD(int32_t, block_tables, bt + key / kPageB);
      const typename Elem<T>::S* vr = v_cache + (page * G + g) * dv * kPageB + key % kPageB;
      const float wj = ws[jj];
#pragma unroll
      for (int i = 0; i < DV_PER_LANE; ++i) {
        const int c = lane + 64 * i;
        if (c < dv) acc[i] += wj * MI355_LDF(T, v_cache, vr + c * kPageB);
      }
    }
    __syncthreads();
  }
  if (sink != nullptr) {                                // one more term in the denominator, no value
    const float sk = MI355_LD(float, sink, sink + h);
    const float mn = fmaxf(m, sk);
    const float corr = expf(m - mn);
    l = l * corr + expf(sk - mn);
#pragma unroll
    for (int i = 0; i < DV_PER_LANE; ++i) acc[i] *= corr;
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < DV_PER_LANE; ++i) {
    const int c = lane + 64 * i;
    if (c >= dv) continue;
    float gt = 1.0f;
    if (gate != nullptr)
      gt = 1.0f / (1.0f + expf(-MI355_LDF(T, gate, gate + t * gate_stride + (gate_per_channel ? h * dv + c : h))));
    MI355_STF(T, out, out + t * out_stride + static_cast<int64_t>(h) * dv + c, acc[i] * inv * gt);
  }
}

// The matrix-core form for 16-bit storage, d a multiple of 32, dv a multiple of 16.  One wave per
// (tile of up to 16 consecutive rows of one chunk, HB query heads of one kv head): K and V fragments
// are loaded once for the HB heads.  Keys go 32 at a time (two pages).  Scores are computed
// transposed, S^T = K Q^T: a lane then holds, for its query (lane % 16), the scores of keys
// 4 (lane / 16) + r of either page -- after the exponential exactly an A-operand fragment of P V, V
// pages being [vdim, 16 tokens].  The softmax runs on line in base 2 (a reference and a sum per query and
// head; the reference follows the running maximum lazily, and accumulators are rescaled only then).  Rows of one tile may
// lie in two blocks: the walk starts at the first row's block and every row masks for itself.
// gridDim.z > 1: the 32-key tiles are dealt out to the z workgroups in turn, each leaves its
// accumulators, maxima and sums in fp32 scratch, and bias_attn_merge_kernel joins them.
// DS / CB: fragment counts the registers are sized for (2 / 4 for heads of up to 64 channels, else
// 4 / 8); PEN: the distance penalty is computed (off: no logarithm per score).
template <typename T, int HB, int DS, int CB, bool PEN>
__global__ __launch_bounds__(256) void softmax_bias_attn_mfma_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q, int64_t q_stride, const uint16_t* __restrict__ k_cache,
    const uint16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tiles, int num_tiles, const int64_t* __restrict__ positions, const float* __restrict__ r1,
    const float* __restrict__ r2, const uint16_t* __restrict__ gate, int64_t gate_stride, int gate_per_channel, int H, int G,
    int d, int dv, int block, int window, float scale, float* __restrict__ part_acc, float* __restrict__ part_ml,
    int64_t total_rows, const float* __restrict__ sink, int64_t out_stride) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  // Workgroups go to the 8 XCDs in turn (x fastest), each XCD with an L2 of its own.  Where the plane of
  // workgroups divides by 8, XCD k takes the k-th eighth of the (head group, tile) pairs in head-major order:
  // the tiles of one kv head then read its K/V through one L2 instead of through all eight.
  int bx = blockIdx.x, by = blockIdx.y;
  const int plane = gridDim.x * gridDim.y;
  if (plane % 8 == 0) {
    const int lin = blockIdx.x + blockIdx.y * gridDim.x;
    const int v = (lin & 7) * (plane >> 3) + (lin >> 3);
    bx = v % gridDim.x;
    by = v / gridDim.x;
  }
  const int tile = bx * (blockDim.x >> 6) + wave;
  if (tile >= num_tiles) return;                        // (no workgroup barrier below)
  const int rep = H / G, hbs = rep / HB;
  const int g = by / hbs, h0 = g * rep + (by % hbs) * HB;
  const int nz = gridDim.z, z = blockIdx.z;
  const int li = lane & 15, kk = lane >> 4;
  const int seq = MI355_LD(int32_t, tiles, tiles + 3 * tile);
  const int64_t row0 = MI355_LD(int32_t, tiles, tiles + 3 * tile + 1);
  const int nrows = MI355_LD(int32_t, tiles, tiles + 3 * tile + 2);
  const int64_t p0 = MI355_LD(int64_t, positions, positions + row0);
  const int32_t* bt = block_tables + static_cast<int64_t>(seq) * max_blocks;
  const int ds = d >> 5, cbs = dv >> 4;
  const int64_t p_last = p0 + nrows - 1;
  const int64_t lo0 = first_visible(p0, block, window);
  const bool valid = li < nrows;
  const int64_t my_p = p0 + li;                         // position of this lane's query
  const int64_t my_lo = first_visible(my_p, block, window);
  uint4 qf[HB][DS];
  float a1[HB], a2[HB], m[HB], l[HB];
  f32x4 acc[HB][CB];
  const float scale2 = scale * kLog2eB;
#pragma unroll
  for (int i = 0; i < HB; ++i) {
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      qf[i][s] = make_uint4(0, 0, 0, 0);
      if (s < ds && valid)
        qf[i][s] = MI355_LD(uint4, q, q + (row0 + li) * q_stride + static_cast<int64_t>(h0 + i) * d + 32 * s + 8 * kk);
    }
    a1[i] = PEN ? MI355_LD(float, r1, r1 + h0 + i) : 0.f;               // ln(x) r1 = log2(x) r1 ln 2, times log2 e again: r1
    a2[i] = PEN ? MI355_LD(float, r2, r2 + h0 + i) : 0.f;
    m[i] = -1.0e30f;
    l[i] = 0.f;
#pragma unroll
    for (int c = 0; c < CB; ++c) acc[i][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // the pages of a tile are looked up one tile ahead: the table's trip to memory then runs beside the
  // current tile's K/V loads instead of in front of the next tile's
  const int64_t first = ((lo0 >> 5) << 5) + 32 * z;
  int32_t pg[2] = {0, 0};
#pragma unroll
  for (int half = 0; half < 2; ++half)
    if (first + 16 * half <= p_last) pg[half] = MI355_LD(int32_t, block_tables, bt + (first + 16 * half) / kPageB);
  for (int64_t base = first; base <= p_last; base += 32 * nz) {
    uint4 kf[2][DS];
    uint2 vf[2][CB];
    int32_t npg[2] = {0, 0};
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int64_t nb = base + 32 * nz + 16 * half;
      if (nb <= p_last) npg[half] = MI355_LD(int32_t, block_tables, bt + nb / kPageB);
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int64_t kb = base + 16 * half;
      const bool have = kb <= p_last;
      const int64_t page = pg[half];
      const uint16_t* kr = k_cache + ((page * G + g) * kPageB + li) * d + 8 * kk;
      const uint16_t* vr = v_cache + ((page * G + g) * dv + li) * kPageB + 4 * kk;
#pragma unroll
      for (int s = 0; s < DS; ++s)
        kf[half][s] = (have && s < ds) ? MI355_LD(uint4, k_cache, kr + 32 * s) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int c = 0; c < CB; ++c)
        vf[half][c] = (have && c < cbs) ? MI355_LD(uint2, v_cache, vr + 16 * c * kPageB) : make_uint2(0, 0);
    }
    if (base + 31 > p_last) {
      // slots past the newest key may hold anything (0 * NaN is NaN): clear them in the last tile
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int64_t k0 = base + 16 * half + 4 * kk;
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          if (k0 > p_last) vf[half][c].x &= 0xFFFF0000u;
          if (k0 + 1 > p_last) vf[half][c].x &= 0x0000FFFFu;
          if (k0 + 2 > p_last) vf[half][c].y &= 0xFFFF0000u;
          if (k0 + 3 > p_last) vf[half][c].y &= 0x0000FFFFu;
        }
      }
    }
    bool vis[2][4];
    float dist[2][4];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int64_t key = base + 16 * half + 4 * kk + r;
        vis[half][r] = valid && key <= my_p && key >= my_lo;
        dist[half][r] = PEN && vis[half][r] ? static_cast<float>(my_p - key) : 0.f;
      }
    }
    uint32_t pw[HB][4];
    float corr[HB];
    bool moved = false;
#pragma unroll
    for (int i = 0; i < HB; ++i) {
      float sc[2][4];
      float tmax = -1.0e30f;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        f32x4 sacc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < DS; ++s)
          if (s < ds) sacc = T::mfma(kf[half][s], qf[i][s], sacc);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // base 2 throughout: q.k scale log2(e) - r1 log2(1 + r2 dist)
          sc[half][r] = sacc[r] * scale2;
          if (PEN) sc[half][r] -= a1[i] * __builtin_amdgcn_logf(1.0f + a2[i] * dist[half][r]);
          if (vis[half][r]) tmax = fmaxf(tmax, sc[half][r]);
        }
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      // The reference of the exponentials follows the maximum only when that grew by more than kLazyLog2:
      // below that the weights of this and later tiles reach 2^kLazyLog2 at most (harmless in fp32 sums and
      // in the 16-bit A operand, whose relative precision does not depend on the magnitude), and the
      // accumulators of all heads are spared a rescale in nearly every tile.
      const float mn = fmaxf(m[i], tmax);
      const bool grow = mn - m[i] > kLazyLog2;
      corr[i] = grow ? __builtin_amdgcn_exp2f(m[i] - mn) : 1.0f;
      if (grow) m[i] = mn;
      l[i] *= corr[i];
      moved |= grow;
      float w[2][4];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          w[half][r] = vis[half][r] ? __builtin_amdgcn_exp2f(sc[half][r] - m[i]) : 0.f;
          l[i] += w[half][r];
        }
      }
      pw[i][0] = T::pack2(w[0][0], w[0][1]);
      pw[i][1] = T::pack2(w[0][2], w[0][3]);
      pw[i][2] = T::pack2(w[1][0], w[1][1]);
      pw[i][3] = T::pack2(w[1][2], w[1][3]);
    }
    // the accumulators hold queries 4 kk + r: their corrections live in the lanes whose li is that query
    if (__any(moved)) {
#pragma unroll
      for (int i = 0; i < HB; ++i) {
        float cr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr[i], 4 * kk + r, 64);
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          if (c < cbs) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][c][r] *= cr[r];
          }
        }
      }
    }
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      if (c < cbs) {
        const uint4 v4 = make_uint4(vf[0][c].x, vf[0][c].y, vf[1][c].x, vf[1][c].y);
#pragma unroll
        for (int i = 0; i < HB; ++i)
          acc[i][c] = T::mfma(make_uint4(pw[i][0], pw[i][1], pw[i][2], pw[i][3]), v4, acc[i][c]);
      }
    }
    pg[0] = npg[0];
    pg[1] = npg[1];
  }
  // C layout: this lane holds rows 4 kk + r of column li of every 16-column block
#pragma unroll
  for (int i = 0; i < HB; ++i) {
    const int h = h0 + i;
    float lt = l[i];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (part_acc != nullptr) {
      if (valid && kk == 0) {
        float* ml = part_ml + ((z * total_rows + row0 + li) * H + h) * 2;
        MI355_ST(float, part_ml, ml, m[i]);
        MI355_ST(float, part_ml, ml + 1, lt);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int rr = 4 * kk + r;
        if (rr >= nrows) continue;
        float* pa = part_acc + ((z * total_rows + row0 + rr) * H + h) * dv + li;
#pragma unroll
        for (int c = 0; c < CB; ++c)
          if (c < cbs) MI355_ST(float, part_acc, pa + 16 * c, acc[i][c][r]);
      }
      continue;
    }
    float f = 1.0f / lt;
    if (sink != nullptr) {
      // the extra term of the denominator, base 2 like the maxima: numerator and denominator are both
      // relative to m[i], so the accumulators only need the ratio
      const float sk = MI355_LD(float, sink, sink + h) * kLog2eB;
      const float mn = fmaxf(m[i], sk);
      const float cm = __builtin_amdgcn_exp2f(m[i] - mn);
      f = cm / (lt * cm + __builtin_amdgcn_exp2f(sk - mn));
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int rr = 4 * kk + r;
      const float fr = __shfl(f, rr, 64);
      if (rr >= nrows) continue;
      const uint16_t* gr = gate != nullptr ? gate + (row0 + rr) * gate_stride + (gate_per_channel ? h * dv : h) : nullptr;
      float gh = 1.0f;
      if (gate != nullptr && !gate_per_channel) gh = 1.0f / (1.0f + expf(-T::to_f(MI355_LD(uint16_t, gate, gr))));
#pragma unroll
      for (int c = 0; c < CB; ++c) {
        if (c >= cbs) continue;
        float gt = gh;
        if (gate != nullptr && gate_per_channel) gt = 1.0f / (1.0f + expf(-T::to_f(MI355_LD(uint16_t, gate, gr + 16 * c + li))));
        MI355_ST(uint16_t, out, out + (row0 + rr) * out_stride + static_cast<int64_t>(h) * dv + 16 * c + li,
                 T::from_f(acc[i][c][r] * fr * gt));
      }
    }
  }
}

// joins the key splits of softmax_bias_attn_mfma_kernel and applies the gate
template <typename T>
__global__ __launch_bounds__(256) void bias_attn_merge_kernel(uint16_t* __restrict__ out, const float* __restrict__ part_acc,
                                                              const float* __restrict__ part_ml,
                                                              const uint16_t* __restrict__ gate, int64_t gate_stride,
                                                              int gate_per_channel, int64_t rows, int H, int dv, int splits,
                                                              const float* __restrict__ sink, int64_t out_stride) {
  const int64_t pairs = rows * H, total = pairs * dv;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t pair = i / dv;
    const int c = static_cast<int>(i % dv);
    const int64_t row = pair / H;
    const int h = static_cast<int>(pair % H);
    float M = -1.0e30f;
    for (int z = 0; z < splits; ++z) M = fmaxf(M, MI355_LD(float, part_ml, part_ml + (z * pairs + pair) * 2));
    float den = 0.f, num = 0.f;
    for (int z = 0; z < splits; ++z) {
      const float* ml = part_ml + (z * pairs + pair) * 2;
      const float e = __builtin_amdgcn_exp2f(MI355_LD(float, part_ml, ml) - M);
      den += MI355_LD(float, part_ml, ml + 1) * e;
      num += MI355_LD(float, part_acc, part_acc + (z * pairs + pair) * dv + c) * e;
    }
    if (sink != nullptr) {
      const float sk = MI355_LD(float, sink, sink + h) * kLog2eB;
      const float mn = fmaxf(M, sk);
      const float cm = __builtin_amdgcn_exp2f(M - mn);
      num *= cm;
      den = den * cm + __builtin_amdgcn_exp2f(sk - mn);
    }
    float v = num / den;
    if (gate != nullptr)
      v /= 1.0f + expf(-T::to_f(MI355_LD(uint16_t, gate, gate + row * gate_stride + (gate_per_channel ? h * dv + c : h))));
    MI355_ST(uint16_t, out, out + row * out_stride + static_cast<int64_t>(h) * dv + c, T::from_f(v));
  }
}

}  // namespace mi355

using namespace mi355;

#define REQ_DTYPE(dtype) MI355_REQUIRE((dtype) >= MI355_BF16 && (dtype) <= MI355_F32, MI355_ERR_UNSUPPORTED, "dtype code %d", (dtype))

extern "C" int32_t mi355_qk_norm_kv_write(void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                          int64_t v_stride, const float* q_weight, const float* k_weight,
                                          const int64_t* slot_mapping, void* k_cache, void* v_cache, int64_t num_tokens,
                                          int32_t num_heads, int32_t num_kv_heads, int32_t head_dim, int32_t v_dim, float eps,
                                          int32_t dtype, void* stream) {
  MI355_REQUIRE(q && k && v && q_weight && k_weight && slot_mapping && k_cache && v_cache, MI355_ERR_INVALID,
                "qk_norm_kv_write: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && num_kv_heads > 0 && head_dim > 0 && v_dim > 0, MI355_ERR_INVALID,
                "qk_norm_kv_write: sizes");
  MI355_REQUIRE(q_stride >= static_cast<int64_t>(num_heads) * head_dim &&
                    k_stride >= static_cast<int64_t>(num_kv_heads) * head_dim &&
                    v_stride >= static_cast<int64_t>(num_kv_heads) * v_dim,
                MI355_ERR_INVALID, "qk_norm_kv_write: row strides shorter than the rows");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((qk_norm_kv_write_kernel<TT>), dim3(num_tokens), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(q), q_stride,
                                                  static_cast<const Elem<TT>::S*>(k), k_stride,
                                                  static_cast<const Elem<TT>::S*>(v), v_stride, q_weight, k_weight,
                                                  slot_mapping, static_cast<Elem<TT>::S*>(k_cache),
                                                  static_cast<Elem<TT>::S*>(v_cache), num_heads, num_kv_heads, head_dim,
                                                  v_dim, eps));
  return check_launch("qk_norm_kv_write");
}

template <typename TT>
static void launch_bias_attn(hipStream_t s, void* out, const void* q, int64_t q_stride, const void* k_cache,
                             const void* v_cache, const int32_t* block_tables, int32_t max_blocks, const int32_t* tok_seq,
                             const int64_t* positions, const float* r1, const float* r2, const void* gate,
                             int64_t gate_stride, int gate_per_channel, int64_t T, int H, int G, int d, int dv, int block,
                             int window, float scale, const float* sink, int64_t out_stride) {
  typedef typename Elem<TT>::S E;
  const dim3 grid(static_cast<unsigned>(T), static_cast<unsigned>(H));
  const size_t lds = (static_cast<size_t>(d) + 64) * sizeof(float);
#define MI355_BATTN(N)                                                                                             \
  hipLaunchKernelGGL((softmax_bias_attn_kernel<TT, N>), grid, dim3(64), lds, s, static_cast<E*>(out),              \
                     static_cast<const E*>(q), q_stride, static_cast<const E*>(k_cache),                           \
                     static_cast<const E*>(v_cache), block_tables, max_blocks, tok_seq, positions, r1, r2,         \
                     static_cast<const E*>(gate), gate_stride, gate_per_channel, H, G, d, dv, block, window, scale, \
                     sink, out_stride)
  if (dv <= 64) MI355_BATTN(1);
  else if (dv <= 128) MI355_BATTN(2);
  else MI355_BATTN(4);
#undef MI355_BATTN
}

extern "C" int64_t mi355_softmax_bias_attn_workspace(int64_t num_tokens, int32_t num_heads, int32_t v_dim, int32_t num_splits) {
  return static_cast<int64_t>(num_splits) * num_tokens * num_heads * (v_dim + 2);          // floats
}

extern "C" int32_t mi355_softmax_bias_attn(void* out, const void* q, int64_t q_stride, const void* k_cache,
                                           const void* v_cache, const int32_t* block_tables, int32_t max_blocks,
                                           const int32_t* tok_seq, const int64_t* positions, const float* r1,
                                           const float* r2, const void* gate, int64_t gate_stride,
                                           int32_t gate_per_channel, int64_t num_tokens, int32_t num_heads,
                                           int32_t num_kv_heads, int32_t head_dim, int32_t v_dim, int32_t block,
                                           int32_t window, float scale, const int32_t* tiles, int32_t num_tiles,
                                           float* workspace, int32_t num_splits, const float* sink, int64_t out_stride,
                                           int32_t dtype, void* stream) {
  MI355_REQUIRE(out && q && k_cache && v_cache && block_tables && tok_seq && positions, MI355_ERR_INVALID,
                "softmax_bias_attn: null pointer");
  MI355_REQUIRE((r1 == nullptr) == (r2 == nullptr), MI355_ERR_INVALID, "softmax_bias_attn: r1 and r2 go together");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0 &&
                    head_dim > 0 && v_dim > 0 && max_blocks > 0 && block >= 0 && window >= 0,
                MI355_ERR_INVALID, "softmax_bias_attn: sizes");
  MI355_REQUIRE(v_dim <= 256 && head_dim <= 8192 && num_heads <= 65535, MI355_ERR_UNSUPPORTED,
                "softmax_bias_attn: v_dim %d (at most 256), head_dim %d", v_dim, head_dim);
  MI355_REQUIRE(gate == nullptr || gate_stride >= (gate_per_channel ? static_cast<int64_t>(num_heads) * v_dim : num_heads),
                MI355_ERR_INVALID, "softmax_bias_attn: gate rows shorter than the gate");
  MI355_REQUIRE(out_stride >= static_cast<int64_t>(num_heads) * v_dim, MI355_ERR_INVALID,
                "softmax_bias_attn: output rows shorter than heads * v_dim");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (tiles != nullptr && num_tiles > 0 && dtype != MI355_F32 && head_dim % 32 == 0 && head_dim <= 128 &&
      v_dim % 16 == 0 && v_dim <= 128 && q_stride % 8 == 0 && aligned16(q) && aligned16(k_cache) && aligned16(v_cache)) {
    const int rep = num_heads / num_kv_heads;
    const bool split = workspace != nullptr && num_splits > 1;
    MI355_REQUIRE(num_splits >= 0 && num_splits <= 64, MI355_ERR_INVALID, "softmax_bias_attn: %d key splits", num_splits);
    const int hb = rep % 4 == 0 ? 4 : rep % 3 == 0 ? 3 : rep % 2 == 0 ? 2 : 1;
    const bool small = head_dim <= 64 && v_dim <= 64;       // half the fragments: registers for a second wave per SIMD
    const int waves = num_tiles < 4 ? num_tiles : 4;                              // a tile per wave
    const dim3 grid(static_cast<unsigned>((num_tiles + waves - 1) / waves), static_cast<unsigned>(num_kv_heads * (rep / hb)),
                    split ? num_splits : 1);
    const dim3 block_dim(64u * static_cast<unsigned>(waves));
    const int64_t pairs = num_tokens * num_heads;
    float* part_acc = split ? workspace : nullptr;
    float* part_ml = split ? workspace + static_cast<int64_t>(num_splits) * pairs * v_dim : nullptr;
#define MI355_BMFMA(TT, HB)                                                                                         \
  do {                                                                                                              \
    if (small && r1 != nullptr) MI355_BMFMA_K(TT, HB, 2, 4, true);                                                  \
    else if (small) MI355_BMFMA_K(TT, HB, 2, 4, false);                                                             \
    else if (r1 != nullptr) MI355_BMFMA_K(TT, HB, 4, 8, true);                                                      \
    else MI355_BMFMA_K(TT, HB, 4, 8, false);                                                                        \
  } while (0)
#define MI355_BMFMA_K(TT, HB, DS, CB, PEN)                                                                          \
  hipLaunchKernelGGL((softmax_bias_attn_mfma_kernel<TT, HB, DS, CB, PEN>), grid, block_dim, 0, s,                   \
                     static_cast<uint16_t*>(out), static_cast<const uint16_t*>(q), q_stride,                        \
                     static_cast<const uint16_t*>(k_cache), static_cast<const uint16_t*>(v_cache), block_tables,    \
                     max_blocks, tiles, num_tiles, positions, r1, r2, static_cast<const uint16_t*>(gate),           \
                     gate_stride, gate_per_channel, num_heads, num_kv_heads, head_dim, v_dim, block, window, scale, \
                     part_acc, part_ml, num_tokens, sink, out_stride)
#define MI355_BMFMA_HB(TT)                                                                                          \
  do {                                                                                                              \
    if (hb == 4) MI355_BMFMA(TT, 4);                                                                                \
    else if (hb == 3) MI355_BMFMA(TT, 3);                                                                           \
    else if (hb == 2) MI355_BMFMA(TT, 2);                                                                           \
    else MI355_BMFMA(TT, 1);                                                                                        \
    if (split) {                                                                                                    \
      const int64_t total = pairs * v_dim;                                                                          \
      hipLaunchKernelGGL((bias_attn_merge_kernel<TT>),                                                              \
                         dim3(static_cast<unsigned>((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256)),      \
                         dim3(256), 0, s, static_cast<uint16_t*>(out), part_acc, part_ml,                           \
                         static_cast<const uint16_t*>(gate), gate_stride, gate_per_channel, num_tokens, num_heads,  \
                         v_dim, num_splits, sink, out_stride);                                                      \
    }                                                                                                               \
  } while (0)
    if (dtype == MI355_BF16) MI355_BMFMA_HB(BF16); else MI355_BMFMA_HB(F16);
#undef MI355_BMFMA_HB
#undef MI355_BMFMA_K
#undef MI355_BMFMA
    return check_launch("softmax_bias_attn (matrix cores)");
  }
  MI355_DISPATCH_DTYPE3(dtype, launch_bias_attn<TT>(s, out, q, q_stride, k_cache, v_cache, block_tables, max_blocks,
                                                   tok_seq, positions, r1, r2, gate, gate_stride, gate_per_channel,
                                                   num_tokens, num_heads, num_kv_heads, head_dim, v_dim, block, window,
                                                   scale, sink, out_stride));
  return check_launch("softmax_bias_attn");
}
