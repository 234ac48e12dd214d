// Grouped-query window attention over paged K/V rows: the cache writer and
// the any-dtype attention kernel.
//
// Cache row of a token (one per layer run): [G heads of D key numbers |
// G heads of Dv value numbers], activation type T (bf16 or fp32).
//
// gqa_prepare_kernel: one block per token.  Optional RMS norm over the WHOLE
// query projection (H*D numbers) and the whole key projection (G*D), each
// with its own weight vector; rotate-half rotary positions on the first
// 2*half entries of every head, angle = fp32(position) * inv_freq[i], cos
// and sin scaled by ``amp``; keys go to the cache row, queries to q_out;
// values are a separate projection or the key projection as it came in.
//
// gqa_attn_kernel: one wave per (token, head), the exactness path (fp32
// activations, odd head sizes).  A row at position p sees key j <= p when
// p - j < window or j < keep; the two key ranges [0, min(keep, lo)) and
// [lo, p] are walked as one list.  Scores, the optional distance-bucket bias
// rel[bucket[p-j], head], the online softmax and the per-head sigmoid gate
// are fp32.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

template <typename T>
__global__ __launch_bounds__(256) void gqa_prepare_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long ldq,
    const T* __restrict__ k, long ldk, const T* __restrict__ v, long ldv,
    const float* __restrict__ qn, const float* __restrict__ kn, float eps,
    const float* __restrict__ inv_freq, int half, float amp,
    const int* __restrict__ positions, T* __restrict__ cache,
    const int* __restrict__ slot_mapping, int H, int G, int D, int Dv) {
  __shared__ float red[8], red2[8];
  const long n = blockIdx.x;
  const int nq = H * D, nk = G * D, nv = G * Dv;
  const T* qr = q + n * ldq;
  const T* kr = k + n * ldk;
  float inv_q = 1.f, inv_k = 1.f;
  if (qn) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq; i += 256) {
      const float f = ldf(qr + i);
      sq += f * f;
    }
    for (int i = threadIdx.x; i < nk; i += 256) {
      const float f = ldf(kr + i);
      sk += f * f;
    }
    sq = block_reduce_sum<4>(sq, red);
    sk = block_reduce_sum<4>(sk, red2);
    inv_q = rsqrtf(sq / nq + eps);
    inv_k = rsqrtf(sk / nk + eps);
  }
  const float pos = (float)positions[n];
  T* crow = cache + (long)slot_mapping[n] * (nk + nv);
  T* qo = q_out + n * nq;
  // queries, then keys: same treatment, different source / weight / target
  for (int part = 0; part < 2; ++part) {
    const T* src = part ? kr : qr;
    const float* wn = part ? kn : qn;
    const float inv = part ? inv_k : inv_q;
    T* dst = part ? crow : qo;
    const int cnt = part ? nk : nq;
    for (int i = threadIdx.x; i < cnt; i += 256) {
      const int d = i % D;
      if (d < half) {
        const int j = i + half;
        const float a = ldf(src + i) * inv * (wn ? wn[i] : 1.f);
        const float b = ldf(src + j) * inv * (wn ? wn[j] : 1.f);
        const float ang = pos * inv_freq[d];
        const float c = cosf(ang) * amp, s = sinf(ang) * amp;
        stf(dst + i, a * c - b * s);
        stf(dst + j, b * c + a * s);
      } else if (d >= 2 * half) {
        stf(dst + i, ldf(src + i) * inv * (wn ? wn[i] : 1.f));
      }
    }
  }
  const T* vr = v ? v + n * ldv : kr;
  for (int i = threadIdx.x; i < nv; i += 256) crow[nk + i] = vr[i];
}

void seq_gqa_prepare_store(torch::Tensor q_out, torch::Tensor q,
                           torch::Tensor k, torch::Tensor v,
                           torch::Tensor q_norm, torch::Tensor k_norm,
                           double eps, torch::Tensor inv_freq, double amp,
                           torch::Tensor positions, torch::Tensor cache,
                           torch::Tensor slot_mapping, int64_t H, int64_t G,
                           int64_t D, int64_t Dv) {
  CHECK_ROWS(q);
  CHECK_ROWS(k);
  CHECK_I32(positions);
  CHECK_I32(slot_mapping);
  const long N = q.size(0);
  const bool has_v = v.defined() && v.numel() > 0;
  const bool has_norm = q_norm.defined() && q_norm.numel() > 0;
  const int half = inv_freq.defined() ? (int)inv_freq.numel() : 0;
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0);
  TORCH_CHECK(q.size(1) == H * D && k.size(0) == N && k.size(1) == G * D);
  TORCH_CHECK(2 * half <= D, "rotated entries exceed the head size");
  TORCH_CHECK(has_v || Dv == D, "keys serve as values only when Dv == D");
  auto ty = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == ty && cache.scalar_type() == ty &&
              q_out.scalar_type() == ty);
  if (has_v) {
    CHECK_ROWS(v);
    TORCH_CHECK(v.size(0) == N && v.size(1) == G * Dv && v.scalar_type() == ty);
  }
  if (has_norm) {
    CHECK_F32(q_norm);
    CHECK_F32(k_norm);
    TORCH_CHECK(q_norm.numel() == H * D && k_norm.numel() == G * D);
  }
  if (half) CHECK_F32(inv_freq);
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == G * (D + Dv), "cache row must be G*(D+Dv)");
  TORCH_CHECK(q_out.is_cuda() && q_out.is_contiguous() &&
              q_out.numel() == N * H * D);
  TORCH_CHECK(positions.numel() == N && slot_mapping.numel() == N);
  if (N == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(ty, { hipLaunchKernelGGL((gqa_prepare_kernel<T>), dim3(N), dim3(256), 0, stream,
      (T*)q_out.data_ptr(), (const T*)q.data_ptr(), q.stride(0),
      (const T*)k.data_ptr(), k.stride(0),
      has_v ? (const T*)v.data_ptr() : nullptr, has_v ? v.stride(0) : 0,
      has_norm ? q_norm.data_ptr<float>() : nullptr,
      has_norm ? k_norm.data_ptr<float>() : nullptr, (float)eps,
      half ? inv_freq.data_ptr<float>() : nullptr, half, (float)amp,
      positions.data_ptr<int>(), (T*)cache.data_ptr(),
      slot_mapping.data_ptr<int>(), (int)H, (int)G, (int)D, (int)Dv); });
  HIP_CHECK_KERNEL();
}

template <typename T, int NCH, int KB>
__global__ __launch_bounds__(64) void gqa_attn_kernel(
    T* __restrict__ out,                // (N, H*Dv)
    const T* __restrict__ q,            // (N, H*D) contiguous
    const T* __restrict__ cache,        // (pages*page_size, G*(D+Dv))
    const int* __restrict__ page_table, int max_pages,
    const int* __restrict__ seq_of_tok, const int* __restrict__ positions,
    const float* __restrict__ rel,      // (rows, H) or null
    const int* __restrict__ dist_bucket,   // (window,) or null
    const T* __restrict__ gate, long ldg,  // (N, H) view or null
    int H, int G, int D, int Dv, int page_size, int window, int keep,
    float scale) {
  const long n = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int g = h / (H / G);
  const int row = G * (D + Dv);
  const int koff = g * D, voff = G * D + g * Dv;
  const int pos = positions[n];
  const int b = seq_of_tok[n];
  const int* ptab = page_table + (long)b * max_pages;
  const int lo = pos - window + 1 > 0 ? pos - window + 1 : 0;
  const int nkeep = keep < lo ? keep : lo;
  const int total = nkeep + (pos - lo + 1);

  float qv[NCH], o[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int d = lane + 64 * c;
    qv[c] = d < D ? ldf(q + (n * H + h) * D + d) : 0.f;
    o[c] = 0.f;
  }
  float m = -INFINITY, l = 0.f;

  for (int i0 = 0; i0 < total; i0 += KB) {
    float vv[KB][NCH], s[KB];
    int jj[KB];
#pragma unroll
    for (int t = 0; t < KB; ++t) {
      const int i = i0 + t < total ? i0 + t : total - 1;
      const int j = i < nkeep ? i : lo + (i - nkeep);
      jj[t] = j;
      const long r0 = ((long)ptab[j / page_size] * page_size + j % page_size) * row;
      float acc = 0.f;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d = lane + 64 * c;
        const float kvv = d < D ? ldf(cache + r0 + koff + d) : 0.f;
        vv[t][c] = d < Dv ? ldf(cache + r0 + voff + d) : 0.f;
        acc += qv[c] * kvv;
      }
      s[t] = acc;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
      for (int t = 0; t < KB; ++t) s[t] += __shfl_xor(s[t], off, WAVE_SIZE);
    }
    float mn = m;
#pragma unroll
    for (int t = 0; t < KB; ++t) {
      s[t] *= scale;
      if (rel) s[t] += rel[(long)dist_bucket[pos - jj[t]] * H + h];
      if (i0 + t < total) mn = fmaxf(mn, s[t]);
    }
    const float corr = expf(m - mn);
    float p[KB];
    float ls = 0.f;
#pragma unroll
    for (int t = 0; t < KB; ++t) {
      p[t] = (i0 + t < total) ? expf(s[t] - mn) : 0.f;
      ls += p[t];
    }
    l = l * corr + ls;
    m = mn;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      float acc = o[c] * corr;
#pragma unroll
      for (int t = 0; t < KB; ++t) acc += p[t] * vv[t][c];
      o[c] = acc;
    }
  }
  float inv = 1.f / l;
  if (gate) inv *= sigmoidf_acc(ldf(gate + n * ldg + h));
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int d = lane + 64 * c;
    if (d < Dv) stf(out + (n * H + h) * Dv + d, o[c] * inv);
  }
}

// shared argument checks of both attention entry points
void gqa_attention_check(torch::Tensor out, torch::Tensor q,
                         torch::Tensor cache, torch::Tensor page_table,
                         torch::Tensor seq_of_tok, torch::Tensor positions,
                         int64_t H, int64_t G, int64_t D, int64_t Dv,
                         int64_t window, int64_t keep_first,
                         torch::Tensor rel, torch::Tensor dist_bucket,
                         torch::Tensor gate) {
  CHECK_I32(page_table); CHECK_I32(seq_of_tok); CHECK_I32(positions);
  const long N = q.size(0);
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0 && window >= 1 &&
              keep_first >= 0);
  TORCH_CHECK(q.is_cuda() && q.is_contiguous() && q.dim() == 2 &&
              q.size(1) == H * D);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 &&
              out.size(0) == N && out.size(1) == H * Dv);
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == G * (D + Dv), "cache row must be G*(D+Dv)");
  auto ty = q.scalar_type();
  TORCH_CHECK(cache.scalar_type() == ty && out.scalar_type() == ty);
  TORCH_CHECK(page_table.dim() == 2 && seq_of_tok.numel() == N &&
              positions.numel() == N);
  const bool has_rel = rel.defined() && rel.numel() > 0;
  if (has_rel) {
    CHECK_F32(rel);
    CHECK_I32(dist_bucket);
    TORCH_CHECK(rel.dim() == 2 && rel.size(1) == H);
    TORCH_CHECK(dist_bucket.numel() >= window && keep_first == 0,
                "the distance table must cover the window");
  }
  if (gate.defined() && gate.numel() > 0) {
    CHECK_ROWS(gate);
    TORCH_CHECK(gate.size(0) == N && gate.size(1) == H &&
                gate.scalar_type() == ty);
  }
}

#define GQA_LAUNCH(NCHV)                                                      \
  hipLaunchKernelGGL((gqa_attn_kernel<T, NCHV, 4>), dim3(N, H), dim3(64), 0,  \
      stream, (T*)out.data_ptr(), (const T*)q.data_ptr(),                     \
      (const T*)cache.data_ptr(), page_table.data_ptr<int>(),                 \
      (int)page_table.size(1), seq_of_tok.data_ptr<int>(),                    \
      positions.data_ptr<int>(), has_rel ? rel.data_ptr<float>() : nullptr,   \
      has_rel ? dist_bucket.data_ptr<int>() : nullptr,                        \
      has_gate ? (const T*)gate.data_ptr() : nullptr,                         \
      has_gate ? gate.stride(0) : 0, (int)H, (int)G, (int)D, (int)Dv,         \
      (int)cache.size(1), (int)window, (int)keep_first, (float)scale)

void seq_gqa_window_attention(torch::Tensor out, torch::Tensor q,
                              torch::Tensor cache, torch::Tensor page_table,
                              torch::Tensor seq_of_tok,
                              torch::Tensor positions, int64_t H, int64_t G,
                              int64_t D, int64_t Dv, int64_t window,
                              int64_t keep_first, torch::Tensor rel,
                              torch::Tensor dist_bucket, torch::Tensor gate,
                              double scale) {
  gqa_attention_check(out, q, cache, page_table, seq_of_tok, positions, H, G,
                      D, Dv, window, keep_first, rel, dist_bucket, gate);
  const int N = q.size(0);
  if (N == 0) return;
  const bool has_rel = rel.defined() && rel.numel() > 0;
  const bool has_gate = gate.defined() && gate.numel() > 0;
  const int nch = (int)((std::max(D, Dv) + 63) / 64);
  TORCH_CHECK(nch <= 8, "head sizes above 512 are not supported");
  auto stream = at::hip::getCurrentHIPStream();
  SEQ_DISPATCH_T(q.scalar_type(), {
    switch (nch) {
      case 1: GQA_LAUNCH(1); break;
      case 2: GQA_LAUNCH(2); break;
      case 3: case 4: GQA_LAUNCH(4); break;
      default: GQA_LAUNCH(8); break;
    }
  });
  HIP_CHECK_KERNEL();
}
