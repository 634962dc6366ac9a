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
// Everything is float32 except the loads of dt_raw, B, C, z and the store of y. The operands of eight tokens are
// loaded, and their steps formed, ahead of the eight dependent state updates.
#include "../serving_common.h"

namespace cai {
namespace serving {

constexpr int SCAN_TB = 8;       // tokens whose operands are loaded (and whose steps are formed) ahead of the recurrence
constexpr int SCAN_CHUNK = 64;   // tokens per chunk of the two-pass form

// MODE 0: a block walks a sequence's whole portion (decode tokens, short portions).
// Long portions are cut into chunks of SCAN_CHUNK tokens that run in parallel, in two passes around a combine step
// (the recurrence is linear in the state, and the decay of a chunk is exp(A * sum of its steps)):
// MODE 1: a chunk from a zero state -> its end state E and the sum of its steps, no output;
// combine: per (sequence, channel, place) the chunks in order, S_in[k] = S; S = exp(A * dtsum[k]) * S + E[k]; the
//          final S is the sequence's new state;
// MODE 2: a chunk again from its true incoming state S_in[k] -> the output.
template <typename T, int RPL, int MODE>
__global__ __launch_bounds__(256) void selective_scan_kernel(
    T* __restrict__ y, const float* __restrict__ x, long xs, const T* __restrict__ dt_raw, long dts,
    const float* __restrict__ A_log, const T* __restrict__ Bm, long bs, const T* __restrict__ Cm, long cs,
    const float* __restrict__ D_skip, const float* __restrict__ dt_bias, const T* __restrict__ z, long zs,
    float* __restrict__ state, long ss, const int* __restrict__ cu, const int* __restrict__ start,
    const int* __restrict__ slots, int C, int S, int LN, const int* __restrict__ chunks, float* __restrict__ carry,
    float* __restrict__ dtsum) {
  // chunks [K, 4] = (sequence, first token, end token, -); carry [K, C, S] holds E after pass 1 and S_in after the
  // combine step; dtsum [K, C]
  int b, lo, hi;
  if (MODE == 0) {
    b = blockIdx.x; lo = cu[b]; hi = cu[b + 1];
  } else {
    b = chunks[4 * blockIdx.x]; lo = chunks[4 * blockIdx.x + 1]; hi = chunks[4 * blockIdx.x + 2];
  }
  const int per = blockDim.x / LN;
  const int c_raw = blockIdx.y * per + threadIdx.x / LN;
  const int part = threadIdx.x % LN;
  const bool live = c_raw < C;
  const int c = live ? c_raw : C - 1;  // idle lanes shadow the last channel and store nothing
  float* st = MODE == 0 ? state + (long)slots[b] * ss + (long)c * S : carry + ((long)blockIdx.x * C + c) * S;
  const bool zero = MODE == 1 || (MODE == 0 && start[b] == 0);
  float A[RPL], Sr[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) {
    const int n = part + r * LN;
    const bool ok = n < S;
    A[r] = ok ? -expf(A_log[(long)c * S + n]) : 0.0f;
    Sr[r] = (ok && !zero) ? st[n] : 0.0f;
  }
  const float dsk = D_skip[c], dbias = dt_bias[c];
  float dt_total = 0.0f;
  for (int t0 = lo; t0 < hi; t0 += SCAN_TB) {
    // everything that does not wait for the state: loads, the softplus step, the decays
    float xv[SCAN_TB], dtv[SCAN_TB], zv[SCAN_TB], Bv[SCAN_TB][RPL], Cv[SCAN_TB][RPL];
#pragma unroll
    for (int i = 0; i < SCAN_TB; ++i) {
      const int t = min(t0 + i, hi - 1);
      xv[i] = x[(long)t * xs + c];
      dtv[i] = ldf(dt_raw + (long)t * dts + c);
      if (MODE != 1) zv[i] = ldf(z + (long)t * zs + c);
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        const int n = min(part + r * LN, S - 1);
        Bv[i][r] = ldf(Bm + (long)t * bs + n);
        if (MODE != 1) Cv[i][r] = ldf(Cm + (long)t * cs + n);
      }
    }
#pragma unroll
    for (int i = 0; i < SCAN_TB; ++i) dtv[i] = softplusf_(dtv[i] + dbias);
#pragma unroll
    for (int i = 0; i < SCAN_TB; ++i) {
      if (t0 + i < hi) {
        const float dx = dtv[i] * xv[i];
        float acc = 0.0f;
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
          if (part + r * LN < S) {
            Sr[r] = expf(dtv[i] * A[r]) * Sr[r] + dx * Bv[i][r];
            if (MODE != 1) acc += Sr[r] * Cv[i][r];
          }
        }
        if (MODE == 1) {
          dt_total += dtv[i];
        } else {
          for (int off = 1; off < LN; off <<= 1) acc += __shfl_xor(acc, off);
          if (part == 0 && live) stf(y + (long)(t0 + i) * C + c, (acc + dsk * xv[i]) * (zv[i] * sigmoidf_(zv[i])));
        }
      }
    }
  }
  if (live && MODE != 2) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int n = part + r * LN;
      if (n < S) st[n] = Sr[r];
    }
    if (MODE == 1 && part == 0) dtsum[(long)blockIdx.x * C + c] = dt_total;
  }
}

// One thread per (sequence, channel, place): the chunks of the sequence in order.
__global__ __launch_bounds__(256) void selective_scan_combine_kernel(
    float* __restrict__ carry, const float* __restrict__ dtsum, const float* __restrict__ A_log,
    float* __restrict__ state, long ss, const int* __restrict__ start, const int* __restrict__ slots,
    const int* __restrict__ seq_chunks, int C, int S) {
  const int b = blockIdx.y;
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)C * S) return;
  const int c = (int)(i / S);
  float* st = state + (long)slots[b] * ss + i;
  const float A = -expf(A_log[i]);
  float Sv = start[b] == 0 ? 0.0f : *st;
  for (int k = seq_chunks[b]; k < seq_chunks[b + 1]; ++k) {
    const long at = (long)k * C * S + i;
    const float e = carry[at];
    carry[at] = Sv;
    Sv = expf(A * dtsum[(long)k * C + c]) * Sv + e;
  }
  *st = Sv;
}

at::Tensor selective_scan(at::Tensor x, at::Tensor dt_raw, at::Tensor A_log, at::Tensor Bm, at::Tensor Cm,
                          at::Tensor D_skip, at::Tensor dt_bias, at::Tensor z, at::Tensor state, at::Tensor cu,
                          at::Tensor start, at::Tensor slots, at::ScalarType out_dtype,
                          c10::optional<at::Tensor> chunks, c10::optional<at::Tensor> seq_chunks) {
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
  // chunks [K, 4] int32 = (sequence, first token, end token, -) in sequence order and seq_chunks [B + 1] = each
  // sequence's range of chunks: the two-pass form for long portions; without them one block walks a whole portion
  const bool chunked = chunks.has_value();
  long K = B;
  at::Tensor carry, dtsum;
  const int* chp = nullptr;
  if (chunked) {
    TORCH_CHECK(seq_chunks.has_value(), "the chunked form needs each sequence's range of chunks");
    check_i32(*chunks, "chunks"); check_i32(*seq_chunks, "seq_chunks");
    TORCH_CHECK(chunks->dim() == 2 && chunks->size(1) == 4 && seq_chunks->numel() == B + 1);
    K = chunks->size(0);
    carry = at::empty({K, C, S}, x.options());
    dtsum = at::empty({K, C}, x.options());
    chp = chunks->data_ptr<int>();
  }
  int threads = 256;  // fewer channels per block when the step has too few blocks to cover the chip
  while (threads > 64 && K * (((long)C * LN + threads - 1) / threads) < 2048) threads >>= 1;
  const dim3 grid((unsigned)K, (unsigned)(((long)C * LN + threads - 1) / threads));
  float* carp = chunked ? carry.data_ptr<float>() : nullptr;
  float* dsp = chunked ? dtsum.data_ptr<float>() : nullptr;
#define SCAN_LAUNCH(RPL_, MODE_)                                                                                       \
  hipLaunchKernelGGL((selective_scan_kernel<T, RPL_, MODE_>), grid, dim3(threads), 0, stream(), ptr<T>(y),             \
                     x.data_ptr<float>(), (long)x.stride(0), ptr<T>(dt_raw), (long)dt_raw.stride(0),                   \
                     al.data_ptr<float>(), ptr<T>(Bm), (long)Bm.stride(0), ptr<T>(Cm), (long)Cm.stride(0),             \
                     dk.data_ptr<float>(), db.data_ptr<float>(), ptr<T>(z), (long)z.stride(0), state.data_ptr<float>(), \
                     (long)state.stride(0), cu.data_ptr<int>(), start.data_ptr<int>(), slots.data_ptr<int>(), C, S, LN, \
                     chp, carp, dsp)
#define SCAN_MODE(MODE_)                  \
  do {                                    \
    if (rpl == 1) SCAN_LAUNCH(1, MODE_);  \
    else if (rpl == 2) SCAN_LAUNCH(2, MODE_); \
    else if (rpl == 4) SCAN_LAUNCH(4, MODE_); \
    else SCAN_LAUNCH(8, MODE_);           \
  } while (0)
  SERVING_DISPATCH_ACT(dt_raw, T, {
    if (!chunked) {
      SCAN_MODE(0);
    } else {
      SCAN_MODE(1);
      hipLaunchKernelGGL(selective_scan_combine_kernel, dim3((unsigned)(((long)C * S + 255) / 256), (unsigned)B), dim3(256),
                         0, stream(), carp, dsp, al.data_ptr<float>(), state.data_ptr<float>(), (long)state.stride(0),
                         start.data_ptr<int>(), slots.data_ptr<int>(), seq_chunks->data_ptr<int>(), C, S);
      SCAN_MODE(2);
    }
  });
#undef SCAN_MODE
#undef SCAN_LAUNCH
  HIP_CHECK_LAST();
  return y;
}

}  // namespace serving
}  // namespace cai
