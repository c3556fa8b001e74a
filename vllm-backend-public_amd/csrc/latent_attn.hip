// Attention through a low-rank latent with a sliding window and a sink in the softmax.
// What is cached per token is the normed latent c [rank] and ONE rotated key part kr [rot] shared by
// all heads, side by side in the engine's 16-token pages: cache [blocks, 16, rank + rot].  Every
// head's unrotated key is Wuk_h c and its value Wuv_h c; the products with Wuk and Wuv are moved out
// of the loop over keys:
//     score(i, j, h) = ((Wuk_h^T qn_i,h) . c_j + qr_i,h . kr_j) * scale
//     out(i, h)      = Wuv_h (sum_j p_ij c_j)
// so the kernel below sees one key / value head of width rank + rot / rank serving all query heads,
// takes the absorbed query ql = Wuk_h^T qn and returns the weighted latent; the caller applies Wuv.
//   latent_kv_write      c = x[:rank] / rms * w (fp32), kr = rotate(x[rank:]), into the page slot
//   latent_window_attn   p_ij = exp(s_ij) / (exp(sink_h) + sum_{j' in window} exp(s_ij')), keys j with
//                        0 <= i - j < window; the query's rotated part is rotated on the way in; the
//                        result is multiplied by sigmoid(gate[i, h])
//   latent_q_pack        the query as the matrix-core form reads it: [absorbed part | rotated part] per
//                        (row, head), contiguous
// Scores, weights, the softmax and its running sums, norms and angles are fp32.
//
// The matrix-core form (16-bit storage, rank a multiple of 16, rank + rot of 8).  All heads of a row
// read the same keys, so the 16 rows of a matrix-core tile are 16 consecutive (row, head) pairs of
// one chunk: a decoded token with 16 heads is one full tile.  Scores are computed transposed, S^T =
// C Q^T, which leaves every lane with eight weights of its own query -- an A-operand fragment of the
// second product P C once the latent's fragment lists the same eight keys.  That second product
// contracts over keys, the first over channels, so the pages hold the latent twice: token-major
// (cache, with the rotated key part) for the scores and channel-major (cache_t [blocks, rank, 16])
// for the weighted sum.  The softmax runs on line (running maximum and sum per query, in base 2);
// with key splits every split writes its unnormalised sums, maximum and sum, and a second launch
// merges them, adds the sink and applies the gate.
#include "common.h"

namespace mi355 {

constexpr int kPageL = MI355_BLOCK_SIZE;

// rotate coordinate j of a vector of `rot` coordinates whose first `dims` are rotated (pairs j, j + dims/2)
template <typename T>
__device__ __forceinline__ float rotated_at(const typename Elem<T>::S* base, const typename Elem<T>::S* v, int j, int dims,
                                            const float* table, const float* cs) {
  const int half = dims >> 1;
  if (j >= dims) return MI355_LDF(T, base, v + j);
  if (j < half) {
    const float c = MI355_LD(float, table, cs + j), s = MI355_LD(float, table, cs + half + j);
    return MI355_LDF(T, base, v + j) * c - MI355_LDF(T, base, v + j + half) * s;
  }
  const int jj = j - half;
  const float c = MI355_LD(float, table, cs + jj), s = MI355_LD(float, table, cs + half + jj);
  return MI355_LDF(T, base, v + j) * c + MI355_LDF(T, base, v + jj) * s;
}

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(typename Elem<T>::S* __restrict__ cache,
                                                              typename Elem<T>::S* __restrict__ cache_t,
                                                              const typename Elem<T>::S* __restrict__ x, int64_t x_stride,
                                                              const float* __restrict__ norm_w,
                                                              const float* __restrict__ cos_sin, int max_pos,
                                                              const int64_t* __restrict__ positions,
                                                              const int64_t* __restrict__ slot_mapping, int rank, int rot,
                                                              int dims, float eps) {
  __shared__ float scratch[32];
  const int64_t t = blockIdx.x;
  const int64_t slot = MI355_LD(int64_t, slot_mapping, slot_mapping + t);
  if (slot < 0) return;                                 // (uniform over the workgroup)
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
  const typename Elem<T>::S* row = x + t * x_stride;
  typename Elem<T>::S* dst = cache + slot * (rank + rot);
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = MI355_LDF(T, x, row + i);
    ss += v * v;
  }
  ss = block_sum32(ss, scratch);
  const float r = 1.0f / sqrtf(ss / static_cast<float>(rank) + eps);
  typename Elem<T>::S* dst_t = cache_t == nullptr ? nullptr : cache_t + (slot / kPageL) * rank * kPageL + slot % kPageL;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float c = MI355_LDF(T, x, row + i) * r * MI355_LD(float, norm_w, norm_w + i);
    MI355_STF(T, cache, dst + i, c);
    if (dst_t != nullptr) MI355_STF(T, cache_t, dst_t + static_cast<int64_t>(i) * kPageL, c);
  }
  const float* cs = cos_sin + p * dims;
  for (int j = threadIdx.x; j < rot; j += blockDim.x)
    MI355_STF(T, cache, dst + rank + j, rotated_at<T>(x, row + rank, j, dims, cos_sin, cs));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// One wave per (packed row, query head).  Keys are taken 64 at a time: every lane scores one key,
// the running maximum and sum are updated, the 64 weights go through LDS, then every lane
// accumulates its channels of the latent over the 64 keys.
template <typename T, int CPL>
__global__ __launch_bounds__(64) void latent_window_attn_kernel(
    typename Elem<T>::S* __restrict__ out, int64_t out_stride, int64_t out_head_stride,
    const typename Elem<T>::S* __restrict__ ql, int64_t ql_stride, int64_t ql_head_stride,
    const typename Elem<T>::S* __restrict__ q, int64_t q_stride, int q_head, int q_rot_off,
    const typename Elem<T>::S* __restrict__ cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int64_t* __restrict__ positions, const float* __restrict__ sink,
    const typename Elem<T>::S* __restrict__ gate, int64_t gate_stride, const float* __restrict__ cos_sin, int max_pos,
    int H, int rank, int rot, int dims, int window, float scale) {
  extern __shared__ float lds[];                        // query [rank + rot] | weights [64]
  float* qs = lds;
  float* ws = lds + rank + rot;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int row_w = rank + rot;
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  if (p >= static_cast<int64_t>(max_blocks) * kPageL) p = static_cast<int64_t>(max_blocks) * kPageL - 1;
  const int32_t* bt = block_tables + static_cast<int64_t>(MI355_LD(int32_t, tok_seq, tok_seq + t)) * max_blocks;
  for (int i = lane; i < rank; i += 64) qs[i] = MI355_LDF(T, ql, ql + t * ql_stride + h * ql_head_stride + i);
  {
    const int64_t pc = p >= max_pos ? max_pos - 1 : p;
    const float* cs = cos_sin + pc * dims;
    const typename Elem<T>::S* qr = q + t * q_stride + static_cast<int64_t>(h) * q_head + q_rot_off;
    for (int j = lane; j < rot; j += 64) qs[rank + j] = rotated_at<T>(q, qr, j, dims, cos_sin, cs);
  }
  float m = MI355_LD(float, sink, sink + h), l = 1.0f;  // the sink: one term exp(sink - m), no key, no value
  float acc[CPL];
#pragma unroll
  for (int i = 0; i < CPL; ++i) acc[i] = 0.f;
  int64_t lo = p - window + 1;
  if (lo < 0) lo = 0;
  __syncthreads();
  for (int64_t base = lo; base <= p; base += 64) {
    const int64_t j = base + lane;
    float s = -__builtin_inff();
    if (j <= p) {
      const int64_t page = MI355_LD(int32_t, block_tables, bt + j / kPageL);
      const typename Elem<T>::S* kr = cache + (page * kPageL + j % kPageL) * row_w;
      float d = 0.f;
      for (int i = 0; i < row_w; ++i) d += qs[i] * MI355_LDF(T, cache, kr + i);
      s = d * scale;
    }
    const float mn = fmaxf(m, wave_max(s));
    const float corr = expf(m - mn);
    const float w = j <= p ? expf(s - mn) : 0.f;
    l = l * corr + wave_sum(w);
    m = mn;
#pragma unroll
    for (int i = 0; i < CPL; ++i) acc[i] *= corr;
    ws[lane] = w;
    __syncthreads();
    const int n = static_cast<int>((p - base + 1) < 64 ? (p - base + 1) : 64);
    for (int jj = 0; jj < n; ++jj) {
      const int64_t key = base + jj;
      const int64_t page = MI355_LD(int32_t, block_tables, bt + key / kPageL);
      const typename Elem<T>::S* vr = cache + (page * kPageL + key % kPageL) * row_w;
      const float wj = ws[jj];
#pragma unroll
      for (int i = 0; i < CPL; ++i) {
        const int c = lane + 64 * i;
        if (c < rank) acc[i] += wj * MI355_LDF(T, cache, vr + c);
      }
    }
    __syncthreads();
  }
  float gt = 1.0f / l;
  if (gate != nullptr) gt /= 1.0f + expf(-MI355_LDF(T, gate, gate + t * gate_stride + h));
#pragma unroll
  for (int i = 0; i < CPL; ++i) {
    const int c = lane + 64 * i;
    if (c < rank) MI355_STF(T, out, out + t * out_stride + h * out_head_stride + c, acc[i] * gt);
  }
}

template <typename T>
__global__ __launch_bounds__(64) void latent_q_pack_kernel(typename Elem<T>::S* __restrict__ qe,
                                                           const typename Elem<T>::S* __restrict__ ql, int64_t ql_stride,
                                                           int64_t ql_head_stride, const typename Elem<T>::S* __restrict__ q,
                                                           int64_t q_stride, int q_head, int q_rot_off,
                                                           const float* __restrict__ cos_sin, int max_pos,
                                                           const int64_t* __restrict__ positions, int H, int rank, int rot,
                                                           int dims) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  typename Elem<T>::S* dst = qe + (t * H + h) * (rank + rot);
  for (int i = lane; i < rank; i += 64)
    MI355_ST(typename Elem<T>::S, qe, dst + i, MI355_LD(typename Elem<T>::S, ql, ql + t * ql_stride + h * ql_head_stride + i));
  int64_t p = MI355_LD(int64_t, positions, positions + t);
  p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
  const float* cs = cos_sin + p * dims;
  const typename Elem<T>::S* qr = q + t * q_stride + static_cast<int64_t>(h) * q_head + q_rot_off;
  for (int j = lane; j < rot; j += 64) MI355_STF(T, qe, dst + rank + j, rotated_at<T>(q, qr, j, dims, cos_sin, cs));
}

constexpr float kLog2e = 1.4426950408889634f;

template <typename T, int DS, int CB>
__global__ __launch_bounds__(256) void latent_window_attn_mfma_kernel(
    uint16_t* __restrict__ out, int64_t out_stride, int64_t out_head_stride, const uint16_t* __restrict__ qe,
    const uint16_t* __restrict__ cache, const uint16_t* __restrict__ cache_t, const int32_t* __restrict__ block_tables,
    int max_blocks, const int32_t* __restrict__ tiles, int num_tiles, const int64_t* __restrict__ positions,
    const float* __restrict__ sink, const uint16_t* __restrict__ gate, int64_t gate_stride, int H, int rank, int rot,
    int window, float scale2, float* __restrict__ part_acc, float* __restrict__ part_ml, int64_t total_pairs) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tile = blockIdx.x * (blockDim.x >> 6) + wave;
  if (tile >= num_tiles) return;                        // (no workgroup barrier below)
  const int nz = gridDim.z, z = blockIdx.z;
  const bool split = part_acc != nullptr;
  const int li = lane & 15, kk = lane >> 4;
  const int seq = MI355_LD(int32_t, tiles, tiles + 3 * tile);
  const int64_t first = MI355_LD(int32_t, tiles, tiles + 3 * tile + 1);
  const int count = MI355_LD(int32_t, tiles, tiles + 3 * tile + 2);
  const int dq = rank + rot, ds = (dq + 31) >> 5, cbs = rank >> 4;
  const int32_t* bt = block_tables + static_cast<int64_t>(seq) * max_blocks;
  const int64_t p_first = MI355_LD(int64_t, positions, positions + first / H);
  const int64_t p_last = MI355_LD(int64_t, positions, positions + (first + count - 1) / H);
  const bool valid = li < count;
  const int64_t my_pair = first + (valid ? li : count - 1);
  const int64_t my_row = my_pair / H;
  const int my_h = static_cast<int>(my_pair % H);
  const int64_t my_p = MI355_LD(int64_t, positions, positions + my_row);
  uint4 qf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s) {
    qf[s] = make_uint4(0, 0, 0, 0);
    if (valid && s < ds && 32 * s + 8 * kk + 8 <= dq) qf[s] = MI355_LD(uint4, qe, qe + my_pair * dq + 32 * s + 8 * kk);
  }
  f32x4 acc[CB];
#pragma unroll
  for (int c = 0; c < CB; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  // running maximum (base-2 exponent) and this lane's share of the running sum of its query; without
  // splits the sink opens both: one term 2^(sink - m) = 1, held by the first of the query's four lanes
  float m = split ? -1.0e30f : MI355_LD(float, sink, sink + my_h) * kLog2e;
  float l = (!split && kk == 0) ? 1.0f : 0.f;
  int64_t lo = p_first - window + 1;
  if (lo < 0) lo = 0;
  for (int64_t base = ((lo >> 5) << 5) + 32 * z; base <= p_last; base += 32 * nz) {
    float sc[2][4];
    int64_t page[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int64_t kb = base + 16 * half;
      const bool have = kb <= p_last;
      page[half] = have ? MI355_LD(int32_t, block_tables, bt + kb / kPageL) : 0;
      const uint16_t* kr = cache + (page[half] * kPageL + li) * dq + 8 * kk;
      uint4 kf[DS];
#pragma unroll
      for (int s = 0; s < DS; ++s)
        kf[s] = (have && s < ds && 32 * s + 8 * kk + 8 <= dq) ? MI355_LD(uint4, cache, kr + 32 * s) : make_uint4(0, 0, 0, 0);
      f32x4 sacc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DS; ++s)
        if (s < ds) sacc = T::mfma(kf[s], qf[s], sacc);
#pragma unroll
      for (int r = 0; r < 4; ++r) sc[half][r] = sacc[r] * scale2;
    }
    bool vis[2][4];
    float tmax = -1.0e30f;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int64_t key = base + 16 * half + 4 * kk + r;
        vis[half][r] = valid && key <= my_p && my_p - key < window;
        if (vis[half][r]) tmax = fmaxf(tmax, sc[half][r]);
      }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float mn = fmaxf(m, tmax);
    const float corr = __builtin_amdgcn_exp2f(m - mn);
    m = mn;
    l *= corr;
    float w[2][4];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        w[half][r] = vis[half][r] ? __builtin_amdgcn_exp2f(sc[half][r] - mn) : 0.f;
        l += w[half][r];
      }
    }
    const uint4 pw = make_uint4(T::pack2(w[0][0], w[0][1]), T::pack2(w[0][2], w[0][3]), T::pack2(w[1][0], w[1][1]),
                                T::pack2(w[1][2], w[1][3]));
    // the accumulators hold queries 4 kk + r: their corrections live in the lanes whose li is that query
    if (__any(corr != 1.0f)) {
      float cr[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr, 4 * kk + r, 64);
#pragma unroll
      for (int c = 0; c < CB; ++c) {
        if (c < cbs) {
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[c][r] *= cr[r];
        }
      }
    }
#pragma unroll
    for (int c0 = 0; c0 < CB; c0 += 8) {
      if (c0 >= cbs) break;
      uint2 vf[2][8];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int64_t kb = base + 16 * half;
        const bool have = kb <= p_last;
        const uint16_t* vr = cache_t + (page[half] * rank + 16 * c0 + li) * kPageL + 4 * kk;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          vf[half][c] = (have && c0 + c < cbs) ? MI355_LD(uint2, cache_t, vr + 16 * c * kPageL) : make_uint2(0, 0);
          // slots past the newest key may hold anything (0 * NaN is NaN): clear them
          const int64_t k0 = kb + 4 * kk;
          if (k0 + 3 > p_last) {
            if (k0 > p_last) vf[half][c].x &= 0xFFFF0000u;
            if (k0 + 1 > p_last) vf[half][c].x &= 0x0000FFFFu;
            if (k0 + 2 > p_last) vf[half][c].y &= 0xFFFF0000u;
            vf[half][c].y &= 0x0000FFFFu;
          }
        }
      }
#pragma unroll
      for (int c = 0; c < 8; ++c)
        if (c0 + c < cbs)
          acc[c0 + c] = T::mfma(pw, make_uint4(vf[0][c].x, vf[0][c].y, vf[1][c].x, vf[1][c].y), acc[c0 + c]);
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (split) {
    if (valid && kk == 0) {
      float* ml = part_ml + (z * total_pairs + first + li) * 2;
      MI355_ST(float, part_ml, ml, m);
      MI355_ST(float, part_ml, ml + 1, l);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int qi = 4 * kk + r;
      if (qi >= count) continue;
      float* pa = part_acc + (z * total_pairs + first + qi) * rank + li;
#pragma unroll
      for (int c = 0; c < CB; ++c)
        if (c < cbs) MI355_ST(float, part_acc, pa + 16 * c, acc[c][r]);
    }
    return;
  }
  float f = 1.0f / l;
  if (gate != nullptr) f /= 1.0f + expf(-T::to_f(MI355_LD(uint16_t, gate, gate + my_row * gate_stride + my_h)));
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int qi = 4 * kk + r;
    const float fr = __shfl(f, qi, 64);
    if (qi >= count) continue;
    const int64_t pair = first + qi;
    uint16_t* po = out + (pair / H) * out_stride + (pair % H) * out_head_stride + li;
#pragma unroll
    for (int c = 0; c < CB; ++c)
      if (c < cbs) MI355_ST(uint16_t, out, po + 16 * c, T::from_f(acc[c][r] * fr));
  }
}

// merges the key splits of latent_window_attn_mfma_kernel: the sink joins the denominator here
template <typename T>
__global__ __launch_bounds__(256) void latent_attn_reduce_kernel(uint16_t* __restrict__ out, int64_t out_stride,
                                                                 int64_t out_head_stride, const float* __restrict__ part_acc,
                                                                 const float* __restrict__ part_ml,
                                                                 const float* __restrict__ sink,
                                                                 const uint16_t* __restrict__ gate, int64_t gate_stride,
                                                                 int64_t total_pairs, int H, int rank, int splits) {
  const int64_t total = total_pairs * rank;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t pair = i / rank;
    const int c = static_cast<int>(i % rank);
    const int64_t row = pair / H;
    const int h = static_cast<int>(pair % H);
    const float s2 = MI355_LD(float, sink, sink + h) * kLog2e;
    float M = s2;
    for (int z = 0; z < splits; ++z) M = fmaxf(M, MI355_LD(float, part_ml, part_ml + (z * total_pairs + pair) * 2));
    float den = __builtin_amdgcn_exp2f(s2 - M), num = 0.f;
    for (int z = 0; z < splits; ++z) {
      const float* ml = part_ml + (z * total_pairs + pair) * 2;
      const float e = __builtin_amdgcn_exp2f(MI355_LD(float, part_ml, ml) - M);
      den += MI355_LD(float, part_ml, ml + 1) * e;
      num += MI355_LD(float, part_acc, part_acc + (z * total_pairs + pair) * rank + c) * e;
    }
    float v = num / den;
    if (gate != nullptr) v /= 1.0f + expf(-T::to_f(MI355_LD(uint16_t, gate, gate + row * gate_stride + h)));
    MI355_ST(uint16_t, out, out + row * out_stride + h * out_head_stride + c, T::from_f(v));
  }
}

}  // namespace mi355

using namespace mi355;

#define REQ_DTYPE(dtype) MI355_REQUIRE((dtype) >= MI355_BF16 && (dtype) <= MI355_F32, MI355_ERR_UNSUPPORTED, "dtype code %d", (dtype))

extern "C" int32_t mi355_latent_kv_write(void* cache, void* cache_t, const void* x, int64_t x_stride, const float* norm_weight,
                                         const float* cos_sin, int32_t max_pos, const int64_t* positions,
                                         const int64_t* slot_mapping, int64_t num_tokens, int32_t rank, int32_t rot,
                                         int32_t rot_dims, float eps, int32_t dtype, void* stream) {
  MI355_REQUIRE(cache && x && norm_weight && cos_sin && positions && slot_mapping, MI355_ERR_INVALID,
                "latent_kv_write: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && rank > 0 && rot >= 0 && max_pos > 0 && x_stride >= rank + rot, MI355_ERR_INVALID,
                "latent_kv_write: sizes");
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, MI355_ERR_INVALID,
                "latent_kv_write: rot_dims %d must be even and at most %d", rot_dims, rot);
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((latent_kv_write_kernel<TT>), dim3(num_tokens), dim3(256), 0, s,
                                                  static_cast<Elem<TT>::S*>(cache), static_cast<Elem<TT>::S*>(cache_t),
                                                  static_cast<const Elem<TT>::S*>(x), x_stride, norm_weight, cos_sin,
                                                  max_pos, positions, slot_mapping, rank, rot, rot_dims, eps));
  return check_launch("latent_kv_write");
}

template <typename TT>
static void launch_latent_attn(hipStream_t s, void* out, int64_t out_stride, int64_t out_head_stride, const void* ql,
                               int64_t ql_stride, int64_t ql_head_stride, const void* q, int64_t q_stride,
                               int q_head, int q_rot_off, const void* cache, const int32_t* block_tables, int max_blocks,
                               const int32_t* tok_seq, const int64_t* positions, const float* sink, const void* gate,
                               int64_t gate_stride, const float* cos_sin, int max_pos, int64_t T, int H, int rank, int rot,
                               int dims, int window, float scale) {
  typedef typename Elem<TT>::S E;
  const dim3 grid(static_cast<unsigned>(T), static_cast<unsigned>(H));
  const size_t lds = (static_cast<size_t>(rank) + rot + 64) * sizeof(float);
#define MI355_LATTN(N)                                                                                              \
  hipLaunchKernelGGL((latent_window_attn_kernel<TT, N>), grid, dim3(64), lds, s, static_cast<E*>(out), out_stride,  \
                     out_head_stride, static_cast<const E*>(ql), ql_stride, ql_head_stride,                         \
                     static_cast<const E*>(q), q_stride, q_head, q_rot_off,                                         \
                     static_cast<const E*>(cache), block_tables, max_blocks, tok_seq, positions, sink,              \
                     static_cast<const E*>(gate), gate_stride, cos_sin, max_pos, H, rank, rot, dims, window, scale)
  if (rank <= 64) MI355_LATTN(1);
  else if (rank <= 128) MI355_LATTN(2);
  else if (rank <= 256) MI355_LATTN(4);
  else MI355_LATTN(8);
#undef MI355_LATTN
}

extern "C" int32_t mi355_latent_window_attn(void* out, int64_t out_stride, int64_t out_head_stride, const void* q_latent,
                                            int64_t q_latent_stride, int64_t q_latent_head_stride, const void* q,
                                            int64_t q_stride, int32_t q_head_width, int32_t q_rot_offset,
                                            const void* cache, const int32_t* block_tables, int32_t max_blocks,
                                            const int32_t* tok_seq, const int64_t* positions, const float* sink,
                                            const void* gate, int64_t gate_stride, const float* cos_sin, int32_t max_pos,
                                            int64_t num_tokens, int32_t num_heads, int32_t rank, int32_t rot,
                                            int32_t rot_dims, int32_t window, float scale, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && q_latent && q && cache && block_tables && tok_seq && positions && sink && cos_sin,
                MI355_ERR_INVALID, "latent_window_attn: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && num_heads <= 65535 && rank > 0 && rot >= 0 && max_blocks > 0 &&
                    window > 0 && max_pos > 0 && q_rot_offset >= 0 && q_head_width >= q_rot_offset + rot,
                MI355_ERR_INVALID, "latent_window_attn: sizes");
  MI355_REQUIRE(rank <= 512 && rot <= 4096, MI355_ERR_UNSUPPORTED, "latent_window_attn: rank %d (at most 512)", rank);
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, MI355_ERR_INVALID,
                "latent_window_attn: rot_dims %d must be even and at most %d", rot_dims, rot);
  MI355_REQUIRE(q_latent_stride >= rank && q_latent_head_stride >= rank && out_stride >= rank && out_head_stride >= rank &&
                    q_stride >= static_cast<int64_t>(num_heads) * q_head_width,
                MI355_ERR_INVALID, "latent_window_attn: strides shorter than the rows");
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_DTYPE3(dtype, launch_latent_attn<TT>(s, out, out_stride, out_head_stride, q_latent, q_latent_stride,
                                                     q_latent_head_stride, q, q_stride, q_head_width,
                                                     q_rot_offset, cache, block_tables, max_blocks, tok_seq, positions,
                                                     sink, gate, gate_stride, cos_sin, max_pos, num_tokens, num_heads,
                                                     rank, rot, rot_dims, window, scale));
  return check_launch("latent_window_attn");
}

extern "C" int32_t mi355_latent_q_pack(void* q_packed, const void* q_latent, int64_t q_latent_stride,
                                       int64_t q_latent_head_stride, const void* q, int64_t q_stride, int32_t q_head_width,
                                       int32_t q_rot_offset, const float* cos_sin, int32_t max_pos,
                                       const int64_t* positions, int64_t num_tokens, int32_t num_heads, int32_t rank,
                                       int32_t rot, int32_t rot_dims, int32_t dtype, void* stream) {
  MI355_REQUIRE(q_packed && q_latent && q && cos_sin && positions, MI355_ERR_INVALID, "latent_q_pack: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && num_heads > 0 && num_heads <= 65535 && rank > 0 && rot >= 0 && max_pos > 0 &&
                    q_rot_offset >= 0 && q_head_width >= q_rot_offset + rot && q_latent_stride >= rank &&
                    q_latent_head_stride >= rank && q_stride >= static_cast<int64_t>(num_heads) * q_head_width,
                MI355_ERR_INVALID, "latent_q_pack: sizes");
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, MI355_ERR_INVALID,
                "latent_q_pack: rot_dims %d must be even and at most %d", rot_dims, rot);
  REQ_DTYPE(dtype);
  if (num_tokens == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(num_tokens), static_cast<unsigned>(num_heads));
  MI355_DISPATCH_DTYPE3(dtype, hipLaunchKernelGGL((latent_q_pack_kernel<TT>), grid, dim3(64), 0, s,
                                                  static_cast<Elem<TT>::S*>(q_packed),
                                                  static_cast<const Elem<TT>::S*>(q_latent), q_latent_stride,
                                                  q_latent_head_stride, static_cast<const Elem<TT>::S*>(q), q_stride,
                                                  q_head_width, q_rot_offset, cos_sin, max_pos, positions, num_heads, rank,
                                                  rot, rot_dims));
  return check_launch("latent_q_pack");
}

extern "C" int32_t mi355_latent_window_attn_tiles(void* out, int64_t out_stride, int64_t out_head_stride,
                                                  const void* q_packed, const void* cache, const void* cache_t,
                                                  const int32_t* block_tables, int32_t max_blocks, const int32_t* tiles,
                                                  int32_t num_tiles, const int64_t* positions, const float* sink,
                                                  const void* gate, int64_t gate_stride, int64_t num_tokens,
                                                  int32_t num_heads, int32_t rank, int32_t rot, int32_t window, float scale,
                                                  float* partial, int32_t num_splits, int32_t dtype, void* stream) {
  MI355_REQUIRE(out && q_packed && cache && cache_t && block_tables && tiles && positions && sink, MI355_ERR_INVALID,
                "latent_window_attn_tiles: null pointer");
  MI355_REQUIRE(num_tokens >= 0 && num_tiles >= 0 && num_heads > 0 && rank > 0 && rot >= 0 && max_blocks > 0 && window > 0 &&
                    out_stride >= rank && out_head_stride >= rank,
                MI355_ERR_INVALID, "latent_window_attn_tiles: sizes");
  MI355_REQUIRE((dtype == MI355_BF16 || dtype == MI355_F16) && rank % 16 == 0 && (rank + rot) % 8 == 0 && rank <= 512 &&
                    rank + rot <= 640 && aligned16(q_packed) && aligned16(cache) && aligned16(cache_t),
                MI355_ERR_UNSUPPORTED,
                "latent_window_attn_tiles: 16-bit storage, rank %d a multiple of 16 up to 512, rank + rot %d of 8 up to 640",
                rank, rank + rot);
  MI355_REQUIRE(num_splits >= 1 && num_splits <= 64 && (num_splits == 1 || partial != nullptr), MI355_ERR_INVALID,
                "latent_window_attn_tiles: %d key splits", num_splits);
  if (num_tokens == 0 || num_tiles == 0) return MI355_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool split = num_splits > 1;
  const int64_t pairs = num_tokens * num_heads;
  float* part_acc = split ? partial : nullptr;
  float* part_ml = split ? partial + static_cast<int64_t>(num_splits) * pairs * rank : nullptr;
  // few tiles (decoded tokens): one wave per workgroup, so that they spread over the compute units
  const int waves = static_cast<int64_t>(num_tiles) * num_splits <= 2048 ? 1 : 4;
  const dim3 grid(static_cast<unsigned>((num_tiles + waves - 1) / waves), 1u, static_cast<unsigned>(num_splits));
  const dim3 block(64u * static_cast<unsigned>(waves));
  const float scale2 = scale * kLog2e;
  const int dq = rank + rot;
#define MI355_LMFMA(TT, DS, CB)                                                                                       \
  hipLaunchKernelGGL((latent_window_attn_mfma_kernel<TT, DS, CB>), grid, block, 0, s, static_cast<uint16_t*>(out),    \
                     out_stride, out_head_stride, static_cast<const uint16_t*>(q_packed),                             \
                     static_cast<const uint16_t*>(cache), static_cast<const uint16_t*>(cache_t), block_tables,        \
                     max_blocks, tiles, num_tiles, positions, sink, static_cast<const uint16_t*>(gate), gate_stride,  \
                     num_heads, rank, rot, window, scale2, part_acc, part_ml, pairs)
#define MI355_LMFMA_SIZES(TT)                                                                                         \
  do {                                                                                                                \
    if (rank <= 64 && dq <= 128) MI355_LMFMA(TT, 4, 4);                                                               \
    else if (rank <= 128 && dq <= 256) MI355_LMFMA(TT, 8, 8);                                                         \
    else if (rank <= 256 && dq <= 384) MI355_LMFMA(TT, 12, 16);                                                       \
    else MI355_LMFMA(TT, 20, 32);                                                                                     \
    if (split) {                                                                                                      \
      const int64_t blocks = (pairs * rank + 255) / 256;                                                              \
      hipLaunchKernelGGL((latent_attn_reduce_kernel<TT>), dim3(static_cast<unsigned>(blocks > 4096 ? 4096 : blocks)), \
                         dim3(256), 0, s, static_cast<uint16_t*>(out), out_stride, out_head_stride, part_acc, part_ml, \
                         sink, static_cast<const uint16_t*>(gate), gate_stride, pairs, num_heads, rank, num_splits);  \
    }                                                                                                                 \
  } while (0)
  if (dtype == MI355_BF16) MI355_LMFMA_SIZES(BF16); else MI355_LMFMA_SIZES(F16);
#undef MI355_LMFMA_SIZES
#undef MI355_LMFMA
  return check_launch("latent_window_attn_tiles");
}
