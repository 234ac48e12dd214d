// Table-routed expert feed-forward for decode-sized batches (bf16, MFMA).
//
// Routing is a table over token ids, so a block finds its expert's rows by
// scanning the batch's (token, choice) slots itself: no host routing, no
// sort, no gather copy, and the launch shape depends only on the batch size
// (capturable in a graph).  Grid = (64-column tile, expert); a block whose
// expert got no row exits at once.  The op is weight-read bound at these
// batch sizes (every live expert streams its matrices once per step), so a
// wave just streams 16 weight rows with 16-byte loads straight into
// v_mfma_f32_16x16x32_bf16 B fragments while the A fragments (<= 16 token
// rows per pass) come from the activations; fp32 accumulation.
//
//   gated : act[slot, j] = silu(x_t . Wg[e][j]) * (x_t . Wu[e][j])
//   plain : y[slot, n]   = act[slot] . Wd[e][n]
// slot = t * top + choice, e = table[token_t][choice].
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "seq_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;

constexpr int MOE_MAX_SLOTS = 1024;

template <bool GATED>
__global__ __launch_bounds__(256) void moe_table_gemm_kernel(
    bf16_t* __restrict__ out,           // (B*top, Nout)
    const bf16_t* __restrict__ x, long ldx,   // gated: (B, K) by token; else (B*top, K) by slot
    const long* __restrict__ tokens,    // (B,)
    const int* __restrict__ table,      // (V, top)
    const bf16_t* __restrict__ w,       // (E, Nw, K): Nw = 2*Nout if gated
    int B, int top, int K, int Nout) {
  __shared__ int slots[MOE_MAX_SLOTS];
  __shared__ int count;
  const int e = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wid = threadIdx.x >> 6;
  const int l15 = lane & 15, lhi = lane >> 4;
  if (threadIdx.x == 0) count = 0;
  __syncthreads();
  const int S = B * top;
  for (int s = threadIdx.x; s < S; s += 256) {
    if (table[tokens[s / top] * top + s % top] == e) slots[atomicAdd(&count, 1)] = s;
  }
  __syncthreads();
  const int cnt = count;
  if (cnt == 0) return;

  const int n = blockIdx.x * 64 + wid * 16 + l15;   // this lane's B column
  const bool nok = n < Nout;
  const long Nw = GATED ? 2L * Nout : Nout;
  const bf16_t* wrow = w + ((long)e * Nw + (nok ? n : 0)) * K + lhi * 8;
  const bf16_t* wrow2 = wrow + (long)Nout * K;       // up rows (gated)

  for (int c0 = 0; c0 < cnt; c0 += 16) {
    const int si = c0 + l15;
    const int slot = si < cnt ? slots[si] : -1;
    const bf16_t* xrow = x + (long)(slot < 0 ? 0 : (GATED ? slot / top : slot)) * ldx + lhi * 8;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
    const i32x4_t zi = {0, 0, 0, 0};
    const bf16x8_t zero = __builtin_bit_cast(bf16x8_t, zi);
#pragma unroll 4
    for (int k0 = 0; k0 < K; k0 += 32) {
      const bf16x8_t a = slot >= 0 ? *reinterpret_cast<const bf16x8_t*>(xrow + k0) : zero;
      const bf16x8_t b = nok ? *reinterpret_cast<const bf16x8_t*>(wrow + k0) : zero;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
      if (GATED) {
        const bf16x8_t b2 = nok ? *reinterpret_cast<const bf16x8_t*>(wrow2 + k0) : zero;
        acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b2, acc2, 0, 0, 0);
      }
    }
    // C layout: row = lhi*4 + r (slot of the pass), col = l15
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int ri = c0 + lhi * 4 + r;
      if (ri < cnt && nok) {
        const float v = GATED ? siluf_acc(acc[r]) * acc2[r] : acc[r];
        out[(long)slots[ri] * Nout + n] = f2bf(v);
      }
    }
  }
}

// y (B*top, width) = table-routed experts on h (B, width); fills ``act``
// (B*top, ff) on the way.
void seq_moe_table_ffn(torch::Tensor y, torch::Tensor act, torch::Tensor h,
                       torch::Tensor tokens, torch::Tensor table,
                       torch::Tensor w_gu, torch::Tensor w_down) {
  CHECK_I32(table);
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.stride(1) == 1 &&
              h.scalar_type() == torch::kBFloat16);
  TORCH_CHECK(tokens.is_cuda() && tokens.dtype() == torch::kInt64 &&
              tokens.is_contiguous());
  TORCH_CHECK(w_gu.is_contiguous() && w_down.is_contiguous() &&
              w_gu.dim() == 3 && w_down.dim() == 3 &&
              w_gu.scalar_type() == torch::kBFloat16 &&
              w_down.scalar_type() == torch::kBFloat16);
  const int B = h.size(0), W = h.size(1), top = table.size(1);
  const int E = w_gu.size(0), ff = w_gu.size(1) / 2;
  TORCH_CHECK(tokens.numel() == B && table.dim() == 2);
  TORCH_CHECK(w_gu.size(2) == W && w_down.size(0) == E &&
              w_down.size(1) == W && w_down.size(2) == ff);
  TORCH_CHECK(W % 32 == 0 && ff % 32 == 0 && h.stride(0) % 8 == 0,
              "expert GEMM needs widths in multiples of 32");
  TORCH_CHECK(B * top <= MOE_MAX_SLOTS, "batch too large for the decode path");
  TORCH_CHECK(act.is_contiguous() && act.scalar_type() == torch::kBFloat16 &&
              act.size(0) == (long)B * top && act.size(1) == ff);
  TORCH_CHECK(y.is_contiguous() && y.scalar_type() == torch::kBFloat16 &&
              y.size(0) == (long)B * top && y.size(1) == W);
  if (B == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  hipLaunchKernelGGL((moe_table_gemm_kernel<true>), dim3((ff + 63) / 64, E),
                     dim3(256), 0, stream, (bf16_t*)act.data_ptr(),
                     (const bf16_t*)h.data_ptr(), h.stride(0),
                     (const long*)tokens.data_ptr<int64_t>(),
                     table.data_ptr<int>(), (const bf16_t*)w_gu.data_ptr(), B,
                     top, W, ff);
  hipLaunchKernelGGL((moe_table_gemm_kernel<false>), dim3((W + 63) / 64, E),
                     dim3(256), 0, stream, (bf16_t*)y.data_ptr(),
                     (const bf16_t*)act.data_ptr(), (long)ff,
                     (const long*)tokens.data_ptr<int64_t>(),
                     table.data_ptr<int>(), (const bf16_t*)w_down.data_ptr(),
                     B, top, ff, W);
  HIP_CHECK_KERNEL();
}
