// Short causal depthwise convolution (optional bias) over a ragged batch, with the last
// K-1 inputs of every sequence carried in a state slot.
//
// Two launches: the outputs (read the slot's tail, write nothing to it), then
// the tail refresh (one thread owns all K-1 entries of a (sequence, channel),
// reads them before it writes), so no element is read and written by
// different threads of one launch.
#include "../serving_common.h"

namespace cai {
namespace serving {

constexpr int MAX_TAPS = 16;

// x element (n, c) at n*xs + c. tail element (slot, r, c) at slot*ts + r*C + c,
// r = 0 oldest .. K-2 the token just before the portion.
template <typename T, typename TO>
__global__ __launch_bounds__(256) void short_conv_kernel(
    TO* __restrict__ y, const T* __restrict__ x, long xs, const float* __restrict__ taps, const float* __restrict__ tail,
    long ts, const int* __restrict__ cu, const int* __restrict__ start, const int* __restrict__ slots,
    const int* __restrict__ tok_seq, int C, int K, int silu, const float* __restrict__ bias) {
  const int n = blockIdx.x;
  const int b = tok_seq[n];
  const int i = n - cu[b];  // index inside the portion
  const bool fresh = start[b] == 0;
  const float* tl = tail + (long)slots[b] * ts;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float acc = bias != nullptr ? bias[c] : 0.0f;
    for (int d = 0; d < K; ++d) {
      float v;
      if (d <= i) v = ldf(x + (long)(n - d) * xs + c);
      else if (!fresh) v = tl[(long)(K - 1 + i - d) * C + c];
      else v = 0.0f;
      acc += taps[c * K + (K - 1 - d)] * v;
    }
    if (silu) acc = acc * sigmoidf_(acc);
    stf(y + (long)n * C + c, acc);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_tail_kernel(
    const T* __restrict__ x, long xs, float* __restrict__ tail, long ts, const int* __restrict__ cu,
    const int* __restrict__ start, const int* __restrict__ slots, int C, int K) {
  const int b = blockIdx.x;
  const int lo = cu[b], cnt = cu[b + 1] - cu[b];
  const bool fresh = start[b] == 0;
  float* tl = tail + (long)slots[b] * ts;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float keep[MAX_TAPS];
#pragma unroll
    for (int r = 0; r < MAX_TAPS; ++r) {
      if (r < K - 1) {
        // entry r of the new tail = element cnt + r of [old tail (K-1), portion (cnt)]
        const int e = cnt + r;
        keep[r] = e < K - 1 ? (fresh ? 0.0f : tl[(long)e * C + c]) : ldf(x + (long)(lo + e - (K - 1)) * xs + c);
      }
    }
#pragma unroll
    for (int r = 0; r < MAX_TAPS; ++r)
      if (r < K - 1) tl[(long)r * C + c] = keep[r];
  }
}

at::Tensor short_conv(at::Tensor x, at::Tensor taps, c10::optional<at::Tensor> tail, at::Tensor cu, at::Tensor start,
                      at::Tensor slots, at::Tensor tok_seq, bool silu, at::ScalarType out_dtype,
                      c10::optional<at::Tensor> bias) {
  check_act(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1, "x must be [N, C] with unit inner stride");
  const long N = x.size(0);
  const int C = (int)x.size(1), K = (int)taps.size(1);
  TORCH_CHECK(taps.dim() == 2 && taps.size(0) == C && K >= 1 && K <= MAX_TAPS, "taps must be [C, K], K <= 16");
  check_i32(cu, "cu"); check_i32(start, "start"); check_i32(slots, "slots"); check_i32(tok_seq, "tok_seq");
  TORCH_CHECK(tok_seq.numel() == N);
  at::Tensor tp = f32c(taps), bs;
  const float* bp = nullptr;
  if (bias.has_value()) {
    bs = f32c(*bias);
    TORCH_CHECK(bs.numel() == C && bs.is_cuda(), "bias must be [C]");
    bp = bs.data_ptr<float>();
  }
  at::Tensor y = at::empty({N, C}, x.options().dtype(out_dtype));
  if (N == 0) return y;
  const float* tlp = nullptr;
  float* tlw = nullptr;
  long ts = 0;
  if (K > 1) {
    TORCH_CHECK(tail.has_value(), "a convolution with more than one tap carries a tail");
    TORCH_CHECK(is_f32(*tail) && tail->dim() == 3 && tail->size(1) == K - 1 && tail->size(2) == C &&
                tail->stride(2) == 1 && tail->stride(1) == C, "tail must be float32 [slots, K-1, C]");
    tlw = tail->data_ptr<float>();
    tlp = tlw;
    ts = tail->stride(0);
  }
  const int B = (int)start.numel();
  const unsigned gy = (unsigned)((C + 255) / 256);
  SERVING_DISPATCH_ACT(x, T, {
    SERVING_DISPATCH_ACT(y, TO, {
      hipLaunchKernelGGL((short_conv_kernel<T, TO>), dim3((unsigned)N, gy), dim3(256), 0, stream(), ptr<TO>(y), ptr<T>(x),
                         (long)x.stride(0), tp.data_ptr<float>(), tlp, ts, cu.data_ptr<int>(), start.data_ptr<int>(),
                         slots.data_ptr<int>(), tok_seq.data_ptr<int>(), C, K, (int)silu, bp);
    });
    if (K > 1)
      hipLaunchKernelGGL(short_conv_tail_kernel<T>, dim3((unsigned)B, gy), dim3(256), 0, stream(), ptr<T>(x),
                         (long)x.stride(0), tlw, ts, cu.data_ptr<int>(), start.data_ptr<int>(), slots.data_ptr<int>(),
                         C, K);
  });
  HIP_CHECK_LAST();
  return y;
}

}  // namespace serving
}  // namespace cai
