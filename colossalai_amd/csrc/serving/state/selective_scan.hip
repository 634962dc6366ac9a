// Selective scan over a ragged batch: a diagonal state-space recurrence with a decay per
// (channel, state place, token) and the state of every sequence carried in its slot.
//
//   dt = softplus(dt_raw[t, c] + dt_bias[c])
//   S[c, n] <- exp(dt * A[c, n]) * S[c, n] + dt * x[t, c] * B[t, n],   A = -exp(A_log)
//   y[t, c] = (sum_n S[c, n] * C[t, n] + D[c] * x[t, c]) * silu(z[t, c])
//
// A block is (sequence, chunk of channels). LN lanes (a power of two) share a channel: lane
// `part` holds the state places part, part + LN, ... (RPL of them, in registers for the whole
// portion), so neighbouring lanes read neighbouring places of the state row, of B and of C; the
// read-out is summed over the LN lanes by shuffles. The state row is read once at the start of the
// portion (taken as zero for a sequence that starts at position 0) and written once at its end.
// Everything is float32 except the loads of dt_raw, B, C, z and the store of y.
#include "../serving_common.h"

namespace cai {
namespace serving {

template <typename T, int RPL>
__global__ __launch_bounds__(256) void selective_scan_kernel(
    T* __restrict__ y, const float* __restrict__ x, long xs, const T* __restrict__ dt_raw, long dts,
    const float* __restrict__ A_log, const T* __restrict__ Bm, long bs, const T* __restrict__ Cm, long cs,
    const float* __restrict__ D_skip, const float* __restrict__ dt_bias, const T* __restrict__ z, long zs,
    float* __restrict__ state, long ss, const int* __restrict__ cu, const int* __restrict__ start,
    const int* __restrict__ slots, int C, int S, int LN) {
  const int b = blockIdx.x;
  const int lo = cu[b], hi = cu[b + 1];
  const int per = blockDim.x / LN;
  const int c_raw = blockIdx.y * per + threadIdx.x / LN;
  const int part = threadIdx.x % LN;
  const bool live = c_raw < C;
  const int c = live ? c_raw : C - 1;  // idle lanes shadow the last channel and store nothing
  float* st = state + (long)slots[b] * ss + (long)c * S;
  const bool fresh = start[b] == 0;
  float A[RPL], Sr[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) {
    const int n = part + r * LN;
    const bool ok = n < S;
    A[r] = ok ? -expf(A_log[(long)c * S + n]) : 0.0f;
    Sr[r] = (ok && !fresh) ? st[n] : 0.0f;
  }
  const float dsk = D_skip[c], dbias = dt_bias[c];
#pragma unroll 2
  for (int t = lo; t < hi; ++t) {
    const float xv = x[(long)t * xs + c];
    const float dt = softplusf_(ldf(dt_raw + (long)t * dts + c) + dbias);
    const float dx = dt * xv;
    float acc = 0.0f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int n = part + r * LN;
      if (n < S) {
        Sr[r] = expf(dt * A[r]) * Sr[r] + dx * ldf(Bm + (long)t * bs + n);
        acc += Sr[r] * ldf(Cm + (long)t * cs + n);
      }
    }
    for (int off = 1; off < LN; off <<= 1) acc += __shfl_xor(acc, off);
    if (part == 0 && live) {
      const float zv = ldf(z + (long)t * zs + c);
      stf(y + (long)t * C + c, (acc + dsk * xv) * (zv * sigmoidf_(zv)));
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int n = part + r * LN;
      if (n < S) st[n] = Sr[r];
    }
  }
}

at::Tensor selective_scan(at::Tensor x, at::Tensor dt_raw, at::Tensor A_log, at::Tensor Bm, at::Tensor Cm,
                          at::Tensor D_skip, at::Tensor dt_bias, at::Tensor z, at::Tensor state, at::Tensor cu,
                          at::Tensor start, at::Tensor slots, at::ScalarType out_dtype) {
  check_act(dt_raw, "dt_raw");
  TORCH_CHECK(x.is_cuda() && is_f32(x) && x.dim() == 2 && x.stride(1) == 1, "x must be float32 [N, C] with dense rows");
  const long N = x.size(0);
  const int C = (int)x.size(1);
  TORCH_CHECK(A_log.dim() == 2 && A_log.size(0) == C, "A_log must be [C, S]");
  const int S = (int)A_log.size(1);
  auto rows_ok = [&](const at::Tensor& t, int cols) {
    return t.is_cuda() && t.dim() == 2 && t.size(0) == N && t.size(1) == cols && t.stride(1) == 1 &&
           t.scalar_type() == dt_raw.scalar_type();
  };
  TORCH_CHECK(rows_ok(dt_raw, C) && rows_ok(z, C) && rows_ok(Bm, S) && rows_ok(Cm, S),
              "dt_raw, z [N, C] and B, C [N, S] share one activation type and have dense rows");
  TORCH_CHECK(out_dtype == dt_raw.scalar_type(), "the result takes the activations' type");
  TORCH_CHECK(state.is_cuda() && is_f32(state) && state.dim() == 3 && state.size(1) == C && state.size(2) == S &&
              state.stride(2) == 1 && state.stride(1) == S, "state must be float32 [slots, C, S] with dense slots");
  check_i32(cu, "cu"); check_i32(start, "start"); check_i32(slots, "slots");
  const int B = (int)start.numel();
  TORCH_CHECK(cu.numel() == B + 1 && slots.numel() == B);
  at::Tensor al = f32c(A_log), dk = f32c(D_skip), db = f32c(dt_bias);
  TORCH_CHECK(dk.numel() == C && db.numel() == C && al.is_cuda() && dk.is_cuda() && db.is_cuda());
  at::Tensor y = at::empty({N, C}, dt_raw.options());
  if (N == 0 || B == 0) return y;
  const int rpl = S <= 4 ? 1 : S <= 8 ? 2 : S <= 32 ? 4 : 8;
  int LN = 1;
  while (LN * rpl < S) LN <<= 1;
  TORCH_CHECK(LN <= 64, "a state row of more than 512 places does not fit the lanes of a wave");
  int threads = 256;  // fewer channels per block when the step has too few blocks to cover the chip
  while (threads > 64 && (long)B * (((long)C * LN + threads - 1) / threads) < 512) threads >>= 1;
  const dim3 grid((unsigned)B, (unsigned)(((long)C * LN + threads - 1) / threads));
#define SCAN_LAUNCH(RPL_)                                                                                              \
  hipLaunchKernelGGL((selective_scan_kernel<T, RPL_>), grid, dim3(threads), 0, stream(), ptr<T>(y), x.data_ptr<float>(), \
                     (long)x.stride(0), ptr<T>(dt_raw), (long)dt_raw.stride(0), al.data_ptr<float>(), ptr<T>(Bm),      \
                     (long)Bm.stride(0), ptr<T>(Cm), (long)Cm.stride(0), dk.data_ptr<float>(), db.data_ptr<float>(),   \
                     ptr<T>(z), (long)z.stride(0), state.data_ptr<float>(), (long)state.stride(0), cu.data_ptr<int>(), \
                     start.data_ptr<int>(), slots.data_ptr<int>(), C, S, LN)
  SERVING_DISPATCH_ACT(dt_raw, T, {
    if (rpl == 1) SCAN_LAUNCH(1);
    else if (rpl == 2) SCAN_LAUNCH(2);
    else if (rpl == 4) SCAN_LAUNCH(4);
    else SCAN_LAUNCH(8);
  });
#undef SCAN_LAUNCH
  HIP_CHECK_LAST();
  return y;
}

}  // namespace serving
}  // namespace cai
