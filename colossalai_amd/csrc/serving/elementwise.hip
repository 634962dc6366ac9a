// Element-wise serving kernels: token shift with carried previous row,
// squared ReLU, gated SiLU / tanh-GELU of a packed tensor, logit soft-cap, ragged
// scatter of keys/values into pages, rotary positions on neighbouring pairs, and
// the write of a latent-attention row (norm + rotation + scatter).
#include "serving_common.h"

namespace cai {
namespace serving {

// One block per token. prev_row = previous token of the same sequence: the
// row above inside a portion, the slot's saved row at a portion's start, zeros
// at position 0. The block of a portion's FIRST token also saves the portion's
// LAST row into the slot, each thread after its own read of the same element,
// so one launch both consumes and refreshes the slot.
template <typename TO>
__global__ __launch_bounds__(256) void token_shift_kernel(
    TO* __restrict__ out, const float* __restrict__ x, const float* __restrict__ mu, float* __restrict__ prev,
    long prev_stride, const int* __restrict__ cu, const int* __restrict__ start, const int* __restrict__ slots,
    const int* __restrict__ tok_seq, int W) {
  const int n = blockIdx.x;
  const int b = tok_seq[n];
  const int first = cu[b], last = cu[b + 1] - 1;
  const float* xr = x + (long)n * W;
  if (n == first) {
    float* pv = prev + (long)slots[b] * prev_stride;
    const bool fresh = start[b] == 0;
    const float* xl = x + (long)last * W;
    for (int w = threadIdx.x; w < W; w += blockDim.x) {
      const float p = fresh ? 0.0f : pv[w];
      const float xv = xr[w];
      const float keep = xl[w];
      stf(out + (long)n * W + w, xv + (p - xv) * mu[w]);
      pv[w] = keep;
    }
  } else {
    const float* xp = xr - W;
    for (int w = threadIdx.x; w < W; w += blockDim.x) {
      const float xv = xr[w];
      stf(out + (long)n * W + w, xv + (xp[w] - xv) * mu[w]);
    }
  }
}

at::Tensor token_shift(at::Tensor x, at::Tensor mu, at::Tensor prev, at::Tensor cu, at::Tensor start,
                       at::Tensor slots, at::Tensor tok_seq, at::ScalarType out_dtype) {
  TORCH_CHECK(x.is_cuda() && is_f32(x) && x.dim() == 2 && x.is_contiguous(), "x must be contiguous float32 [N, W]");
  TORCH_CHECK(is_f32(prev) && prev.dim() == 2 && prev.size(1) == x.size(1) && prev.stride(1) == 1,
              "prev must be float32 [slots, W] with unit inner stride");
  check_i32(cu, "cu"); check_i32(start, "start"); check_i32(slots, "slots"); check_i32(tok_seq, "tok_seq");
  const long N = x.size(0);
  const int W = (int)x.size(1);
  TORCH_CHECK(tok_seq.numel() == N && cu.numel() == start.numel() + 1 && slots.numel() == start.numel());
  at::Tensor muf = f32c(mu);
  TORCH_CHECK(muf.numel() == W);
  at::Tensor out = at::empty({N, W}, x.options().dtype(out_dtype));
  if (N == 0) return out;
  SERVING_DISPATCH_ACT(out, T, {
    hipLaunchKernelGGL(token_shift_kernel<T>, dim3((unsigned)N), dim3(256), 0, stream(), ptr<T>(out),
                       x.data_ptr<float>(), muf.data_ptr<float>(), prev.data_ptr<float>(), (long)prev.stride(0),
                       cu.data_ptr<int>(), start.data_ptr<int>(), slots.data_ptr<int>(), tok_seq.data_ptr<int>(), W);
  });
  HIP_CHECK_LAST();
  return out;
}

template <typename T>
__global__ __launch_bounds__(256) void relu_squared_kernel(T* __restrict__ out, const T* __restrict__ in, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    // the square is taken of the value as the activation type holds it
    const float v = fmaxf(ldf(in + i), 0.0f);
    stf(out + i, v * v);
  }
}

at::Tensor relu_squared(at::Tensor x) {
  check_act(x, "x");
  TORCH_CHECK(x.is_contiguous());
  at::Tensor out = at::empty_like(x);
  const long n = x.numel();
  if (n == 0) return out;
  SERVING_DISPATCH_ACT(x, T, {
    hipLaunchKernelGGL(relu_squared_kernel<T>, dim3(capped_grid((n + 255) / 256, 4096)), dim3(256), 0, stream(),
                       ptr<T>(out), ptr<T>(x), n);
  });
  HIP_CHECK_LAST();
  return out;
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ out, const float* __restrict__ in, float cap,
                                                      long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    out[i] = cap * tanhf(in[i] / cap);
}

at::Tensor softcap(at::Tensor x, double cap) {
  TORCH_CHECK(x.is_cuda() && is_f32(x) && x.is_contiguous(), "x must be contiguous float32");
  at::Tensor out = at::empty_like(x);
  const long n = x.numel();
  if (n == 0) return out;
  hipLaunchKernelGGL(softcap_kernel, dim3(capped_grid((n + 255) / 256, 4096)), dim3(256), 0, stream(),
                     out.data_ptr<float>(), x.data_ptr<float>(), (float)cap, n);
  HIP_CHECK_LAST();
  return out;
}

// k [N, G*D] / v [N, G*Dv] rows (row-strided) -> pool rows rows[n].
template <typename TI, typename TP>
__global__ __launch_bounds__(256) void paged_kv_write_kernel(
    TP* __restrict__ kpool, TP* __restrict__ vpool, const TI* __restrict__ k, const TI* __restrict__ v, long k_stride,
    long v_stride, const int* __restrict__ rows, int KW, int VW) {
  const int n = blockIdx.x;
  const long r = rows[n];
  for (int i = threadIdx.x; i < KW; i += blockDim.x) stf(kpool + r * KW + i, ldf(k + (long)n * k_stride + i));
  for (int i = threadIdx.x; i < VW; i += blockDim.x) stf(vpool + r * VW + i, ldf(v + (long)n * v_stride + i));
}

void paged_kv_write(at::Tensor k, at::Tensor v, at::Tensor kpool, at::Tensor vpool, at::Tensor rows) {
  check_act(k, "k"); check_act(v, "v");
  TORCH_CHECK(k.dim() == 3 && v.dim() == 3 && kpool.dim() == 4 && vpool.dim() == 4);
  TORCH_CHECK(kpool.is_contiguous() && vpool.is_contiguous() && kpool.scalar_type() == vpool.scalar_type());
  TORCH_CHECK(k.scalar_type() == v.scalar_type() && k.scalar_type() == kpool.scalar_type(),
              "keys, values and pools share one dtype");
  check_i32(rows, "rows");
  const long N = k.size(0);
  const int KW = (int)(k.size(1) * k.size(2)), VW = (int)(v.size(1) * v.size(2));
  TORCH_CHECK(v.size(0) == N && rows.numel() == N);
  TORCH_CHECK(kpool.size(2) * kpool.size(3) == KW && vpool.size(2) * vpool.size(3) == VW, "pool row width mismatch");
  TORCH_CHECK(k.stride(2) == 1 && k.stride(1) == k.size(2) && v.stride(2) == 1 && v.stride(1) == v.size(2),
              "k/v rows must be dense (row stride free)");
  if (N == 0) return;
  SERVING_DISPATCH_ACT(k, T, {
    hipLaunchKernelGGL((paged_kv_write_kernel<T, T>), dim3((unsigned)N), dim3(256), 0, stream(), ptr<T>(kpool),
                       ptr<T>(vpool), ptr<T>(k), ptr<T>(v), (long)k.stride(0), (long)v.stride(0),
                       rows.data_ptr<int>(), KW, VW);
  });
  HIP_CHECK_LAST();
}

// packed [N, 2F] = [gate | up], rows strided by ps -> out [N, F] = silu(gate) * up, formed in float32.
// VEC: eight elements per thread (F and the row stride are multiples of 8 and the base is aligned).
// ACT: 0 = silu(g) = g * sigmoid(g); 1 = the tanh form of GELU, 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))).
template <int ACT>
DEV_INLINE float gate_act(float g) {
  if (ACT == 0) return g * sigmoidf_(g);
  return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
}

template <typename T, bool VEC, int ACT>
__global__ __launch_bounds__(256) void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ packed, long ps,
                                                       long N, int F) {
  constexpr int PER = VEC ? 8 : 1;
  const long total = N * F / PER;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long n = i * PER / F;
    const int f = (int)(i * PER % F);
    if (VEC) {
      float g[8], u[8];
      load8(packed + n * ps + f, g);
      load8(packed + n * ps + F + f, u);
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = gate_act<ACT>(g[e]) * u[e];
      store8(out + n * F + f, g);
    } else {
      const float g = ldf(packed + n * ps + f), u = ldf(packed + n * ps + F + f);
      stf(out + i, gate_act<ACT>(g) * u);
    }
  }
}

template <int ACT>
static at::Tensor gated_act_mul(at::Tensor packed) {
  check_act(packed, "packed");
  TORCH_CHECK(packed.dim() == 2 && packed.stride(1) == 1 && packed.size(1) % 2 == 0, "packed must be [N, 2F] with dense rows");
  const long N = packed.size(0);
  const int F = (int)(packed.size(1) / 2);
  at::Tensor out = at::empty({N, F}, packed.options());
  if (N * F == 0) return out;
  const bool vec = F % 8 == 0 && packed.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(packed.data_ptr()) % 32 == 0;
  SERVING_DISPATCH_ACT(packed, T, {
    if (vec)
      hipLaunchKernelGGL((silu_mul_kernel<T, true, ACT>), dim3(capped_grid((N * F / 8 + 255) / 256, 8192)), dim3(256), 0, stream(),
                         ptr<T>(out), ptr<T>(packed), (long)packed.stride(0), N, F);
    else
      hipLaunchKernelGGL((silu_mul_kernel<T, false, ACT>), dim3(capped_grid((N * F + 255) / 256, 4096)), dim3(256), 0, stream(),
                         ptr<T>(out), ptr<T>(packed), (long)packed.stride(0), N, F);
  });
  HIP_CHECK_LAST();
  return out;
}

at::Tensor silu_mul(at::Tensor packed) { return gated_act_mul<0>(packed); }
at::Tensor gelu_tanh_mul(at::Tensor packed) { return gated_act_mul<1>(packed); }

// ------------------------------------------------------------ rotary on pairs
// The pair (2i, 2i + 1), i < half, of a vector at position p turns by a = p * freqs[i], float32.
DEV_INLINE void turn_pair(float u, float v, float a, float& ou, float& ov) {
  float sn, cs;
  sincosf(a, &sn, &cs);
  ou = u * cs - v * sn;
  ov = v * cs + u * sn;
}

// x element (n, h, r) at n*xs + h*xh + r; out likewise with its own strides. One thread per pair
// (or single trailing channel when R is odd); channels from 2 * half on are copied.
template <typename T>
__global__ __launch_bounds__(256) void rotate_pairs_kernel(
    T* __restrict__ out, long os, long oh, const T* __restrict__ x, long xs, long xh, const int* __restrict__ positions,
    const float* __restrict__ freqs, long N, int H, int R, int half) {
  const int per = (R + 1) / 2;
  const long total = N * H * per;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const int j = (int)(i % per);
    const long nh = i / per;
    const int h = (int)(nh % H);
    const long n = nh / H;
    const T* src = x + n * xs + h * xh + 2 * j;
    T* dst = out + n * os + h * oh + 2 * j;
    const float u = ldf(src);
    if (2 * j + 1 >= R) {
      stf(dst, u);
      continue;
    }
    const float v = ldf(src + 1);
    if (j < half) {
      float ou, ov;
      turn_pair(u, v, (float)positions[n] * freqs[j], ou, ov);
      stf(dst, ou);
      stf(dst + 1, ov);
    } else {
      stf(dst, u);
      stf(dst + 1, v);
    }
  }
}

void rotate_pairs(at::Tensor x, at::Tensor positions, at::Tensor freqs, at::Tensor out) {
  check_act(x, "x"); check_act(out, "out");
  TORCH_CHECK(x.dim() == 3 && out.dim() == 3 && x.sizes() == out.sizes() && x.scalar_type() == out.scalar_type());
  TORCH_CHECK(x.stride(2) == 1 && out.stride(2) == 1, "channels must have unit stride");
  check_i32(positions, "positions");
  const long N = x.size(0);
  const int H = (int)x.size(1), R = (int)x.size(2);
  TORCH_CHECK(positions.numel() == N);
  TORCH_CHECK(freqs.is_cuda() && is_f32(freqs) && freqs.is_contiguous() && 2 * freqs.numel() <= R,
              "freqs must be float32 [dims / 2] with dims <= R");
  if (N * H * R == 0) return;
  const long total = N * H * ((R + 1) / 2);
  SERVING_DISPATCH_ACT(x, T, {
    hipLaunchKernelGGL(rotate_pairs_kernel<T>, dim3(capped_grid((total + 255) / 256, 8192)), dim3(256), 0, stream(),
                       ptr<T>(out), (long)out.stride(0), (long)out.stride(1), ptr<T>(x), (long)x.stride(0),
                       (long)x.stride(1), positions.data_ptr<int>(), freqs.data_ptr<float>(), N, H, R,
                       (int)freqs.numel());
  });
  HIP_CHECK_LAST();
}

// ------------------------------------------------------------- latent row write
// One wave per token: dkv row [rank + R] (row-strided) -> pool row rows[n]: the first `rank`
// channels RMS-normed with a weight (float32 statistics), the last R rotated pair-wise (the
// first 2 * half of them) by the token's position.
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(
    T* __restrict__ pool, const T* __restrict__ dkv, long ds, const float* __restrict__ w,
    const float* __restrict__ freqs, const int* __restrict__ positions, const int* __restrict__ rows, long N, int rank,
    int R, int half, float eps) {
  const int lane = threadIdx.x & 63;
  const long n = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (n >= N) return;
  const T* src = dkv + n * ds;
  T* dst = pool + (long)rows[n] * (rank + R);
  float ssq = 0.0f;
#pragma unroll 4
  for (int i = lane; i < rank; i += 64) {
    const float v = ldf(src + i);
    ssq += v * v;
  }
  ssq = wave_reduce_sum(ssq);
  const float inv = 1.0f / sqrtf(ssq / (float)rank + eps);
#pragma unroll 4
  for (int i = lane; i < rank; i += 64) stf(dst + i, ldf(src + i) * inv * w[i]);
  const float p = (float)positions[n];
  for (int j = lane; 2 * j < R; j += 64) {
    const float u = ldf(src + rank + 2 * j);
    if (2 * j + 1 >= R) {
      stf(dst + rank + 2 * j, u);
      continue;
    }
    float v = ldf(src + rank + 2 * j + 1), ou = u, ov = v;
    if (j < half) turn_pair(u, v, p * freqs[j], ou, ov);
    stf(dst + rank + 2 * j, ou);
    stf(dst + rank + 2 * j + 1, ov);
  }
}

void latent_kv_write(at::Tensor dkv, at::Tensor norm_w, double eps, at::Tensor freqs, at::Tensor positions,
                     at::Tensor pool, at::Tensor rows) {
  check_act(dkv, "dkv");
  TORCH_CHECK(dkv.dim() == 2 && dkv.stride(1) == 1, "dkv must be [N, rank + R] with unit inner stride");
  TORCH_CHECK(pool.is_cuda() && pool.is_contiguous() && pool.dim() == 4 && pool.size(2) == 1 &&
              pool.size(3) == dkv.size(1) && pool.scalar_type() == dkv.scalar_type(),
              "pool must be contiguous [pages, page, 1, rank + R] of dkv's dtype");
  check_i32(positions, "positions"); check_i32(rows, "rows");
  const long N = dkv.size(0);
  at::Tensor w = f32c(norm_w);
  const int rank = (int)w.numel(), R = (int)dkv.size(1) - rank;
  TORCH_CHECK(rank > 0 && R >= 0 && positions.numel() == N && rows.numel() == N);
  TORCH_CHECK(freqs.is_cuda() && is_f32(freqs) && freqs.is_contiguous() && 2 * freqs.numel() <= R,
              "freqs must be float32 [dims / 2] with dims <= R");
  if (N == 0) return;
  SERVING_DISPATCH_ACT(dkv, T, {
    hipLaunchKernelGGL(latent_kv_write_kernel<T>, dim3((unsigned)((N + 3) / 4)), dim3(256), 0, stream(), ptr<T>(pool),
                       ptr<T>(dkv), (long)dkv.stride(0), w.data_ptr<float>(), freqs.data_ptr<float>(),
                       positions.data_ptr<int>(), rows.data_ptr<int>(), N, rank, R, (int)freqs.numel(), (float)eps);
  });
  HIP_CHECK_LAST();
}

// --------------------------------------------- rotate-half rotary + weightless per-head RMS norm
// One wave per (token, head): channel i < half pairs with channel i + half and turns by
// positions[n] * freqs[i] (float32 angle); channels from 2 * half on pass. Then, with eps >= 0, the
// head's vector is divided by sqrt(mean(x^2) + eps) over all D channels. The head's vector stays in
// registers (D <= 64 * PER) between the two steps. x element (n, h, d) at n*xs + h*D + d; out dense.
template <typename T, typename TO, int PER>
__global__ __launch_bounds__(256) void rotate_halves_unit_norm_kernel(
    TO* __restrict__ out, const T* __restrict__ x, long xs, const int* __restrict__ positions,
    const float* __restrict__ freqs, long units, int H, int D, int half, float eps) {
  const int lane = threadIdx.x & 63;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= units) return;
  const long n = unit / H;
  const int h = (int)(unit % H);
  const T* src = x + n * xs + (long)h * D;
  const float p = (float)positions[n];
  float v[PER];
  float ssq = 0.0f;
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int d = lane + 64 * r;
    v[r] = 0.0f;
    if (d < D) {
      const float own = ldf(src + d);
      if (d < 2 * half) {
        const int i = d < half ? d : d - half;
        const float other = ldf(src + (d < half ? d + half : d - half));
        float sn, cs;
        sincosf(p * freqs[i], &sn, &cs);
        v[r] = d < half ? own * cs - other * sn : own * cs + other * sn;
      } else {
        v[r] = own;
      }
      ssq += v[r] * v[r];
    }
  }
  float inv = 1.0f;
  if (eps >= 0.0f) inv = 1.0f / sqrtf(wave_reduce_sum(ssq) / (float)D + eps);
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int d = lane + 64 * r;
    if (d < D) stf(out + unit * D + d, v[r] * inv);
  }
}

at::Tensor rotate_halves_unit_norm(at::Tensor x, at::Tensor positions, c10::optional<at::Tensor> freqs, double eps,
                                   at::ScalarType out_dtype) {
  check_act(x, "x");
  TORCH_CHECK(x.dim() == 3 && x.stride(2) == 1 && (x.size(1) == 1 || x.stride(1) == x.size(2)),
              "x must be [N, H, D] with the heads of a token side by side");
  check_i32(positions, "positions");
  const long N = x.size(0);
  const int H = (int)x.size(1), D = (int)x.size(2);
  TORCH_CHECK(positions.numel() == N && D <= 512, "head sizes up to 512");
  int half = 0;
  const float* fp = nullptr;
  at::Tensor fr;
  if (freqs.has_value() && freqs->numel() > 0) {
    fr = *freqs;
    TORCH_CHECK(fr.is_cuda() && is_f32(fr) && fr.is_contiguous() && 2 * fr.numel() <= D,
                "freqs must be float32 [dims / 2] with dims <= D");
    half = (int)fr.numel();
    fp = fr.data_ptr<float>();
  }
  TORCH_CHECK(out_dtype == at::kFloat || out_dtype == at::kBFloat16);
  at::Tensor out = at::empty({N, H, D}, x.options().dtype(out_dtype));
  const long units = N * H;
  if (units == 0) return out;
  const dim3 grid((unsigned)((units + 3) / 4));
#define RH_LAUNCH(PER_)                                                                                                 hipLaunchKernelGGL((rotate_halves_unit_norm_kernel<T, TO, PER_>), grid, dim3(256), 0, stream(), ptr<TO>(out),                           ptr<T>(x), (long)x.stride(0), positions.data_ptr<int>(), fp, units, H, D, half, (float)eps)
  SERVING_DISPATCH_ACT(x, T, {
    SERVING_DISPATCH_ACT(out, TO, {
      if (D <= 64) RH_LAUNCH(1);
      else if (D <= 128) RH_LAUNCH(2);
      else if (D <= 256) RH_LAUNCH(4);
      else RH_LAUNCH(8);
    });
  });
#undef RH_LAUNCH
  HIP_CHECK_LAST();
  return out;
}

// ------------------------------------------------------------------ value mixing
// out[n, c] = (1 - lam) * a[n, c] + lam * b[n, c], float32 inside, one rounding; rows may be strided.
template <typename T>
__global__ __launch_bounds__(256) void lerp_rows_kernel(T* __restrict__ out, const T* __restrict__ a, long as,
                                                        const T* __restrict__ b, long bs, float lam, long N, int C) {
  const long total = N * C;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long n = i / C;
    const int c = (int)(i % C);
    const float av = ldf(a + n * as + c), bv = ldf(b + n * bs + c);
    stf(out + i, (1.0f - lam) * av + lam * bv);
  }
}

at::Tensor lerp_rows(at::Tensor a, at::Tensor b, double lam) {
  check_act(a, "a"); check_act(b, "b");
  TORCH_CHECK(a.dim() == 2 && b.dim() == 2 && a.sizes() == b.sizes() && a.scalar_type() == b.scalar_type() &&
              a.stride(1) == 1 && b.stride(1) == 1, "a and b must be [N, C] of one type with dense rows");
  const long N = a.size(0);
  const int C = (int)a.size(1);
  at::Tensor out = at::empty({N, C}, a.options());
  if (N * C == 0) return out;
  SERVING_DISPATCH_ACT(a, T, {
    hipLaunchKernelGGL(lerp_rows_kernel<T>, dim3(capped_grid((N * C + 255) / 256, 8192)), dim3(256), 0, stream(),
                       ptr<T>(out), ptr<T>(a), (long)a.stride(0), ptr<T>(b), (long)b.stride(0), (float)lam, N, C);
  });
  HIP_CHECK_LAST();
  return out;
}

// --------------------------------------------------------------- talking heads
// o [N, H, G, Dv] float32 holds every query head's softmax weights applied to every key/value head's
// values; mixing the weights of the heads is linear, so out[n, h, :] = sum_g talk[h, g] * o[n, g, kv(h), :]
// with kv(h) = h / (H / G).
// One thread per (token, kv head c, run of RT heads of group c, channel): it reads the H cross outputs of its place
// once and forms the rows of its RT heads (R = H / G heads in the group). RT = 8 reads the input once per eight heads
// (large steps); RT = 1 gives a small step more threads.
template <typename TO, int RT>
__global__ __launch_bounds__(256) void talk_mix_kernel(TO* __restrict__ out, const float* __restrict__ o,
                                                       const float* __restrict__ talk, long N, int H, int G, int Dv) {
  const int R = H / G, runs = (R + RT - 1) / RT;
  const long total = N * G * runs * Dv;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const int d = (int)(i % Dv);
    const int r0 = (int)(i / Dv % runs) * RT;
    const int c = (int)(i / Dv / runs % G);
    const long n = i / Dv / runs / G;
    float acc[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[r] = 0.0f;
    for (int g = 0; g < H; ++g) {
      const float v = o[((n * H + g) * G + c) * Dv + d];
#pragma unroll
      for (int r = 0; r < RT; ++r)
        if (r0 + r < R) acc[r] += talk[(c * R + r0 + r) * H + g] * v;
    }
#pragma unroll
    for (int r = 0; r < RT; ++r)
      if (r0 + r < R) stf(out + (n * H + c * R + r0 + r) * Dv + d, acc[r]);
  }
}

at::Tensor talk_mix(at::Tensor o, at::Tensor talk, at::ScalarType out_dtype) {
  TORCH_CHECK(o.is_cuda() && is_f32(o) && o.dim() == 4 && o.is_contiguous(), "o must be contiguous float32 [N, H, G, Dv]");
  const long N = o.size(0);
  const int H = (int)o.size(1), G = (int)o.size(2), Dv = (int)o.size(3);
  at::Tensor tk = f32c(talk);
  TORCH_CHECK(tk.is_cuda() && tk.dim() == 2 && tk.size(0) == H && tk.size(1) == H && H % G == 0);
  TORCH_CHECK(out_dtype == at::kFloat || out_dtype == at::kBFloat16);
  at::Tensor out = at::empty({N, H, Dv}, o.options().dtype(out_dtype));
  if (N == 0) return out;
  const bool wide = N * H * Dv >= (1L << 20);
  const long threads = wide ? N * G * ((H / G + 7) / 8) * Dv : N * H * Dv;
  SERVING_DISPATCH_ACT(out, TO, {
    if (wide)
      hipLaunchKernelGGL((talk_mix_kernel<TO, 8>), dim3(capped_grid((threads + 255) / 256, 8192)), dim3(256), 0, stream(),
                         ptr<TO>(out), o.data_ptr<float>(), tk.data_ptr<float>(), N, H, G, Dv);
    else
      hipLaunchKernelGGL((talk_mix_kernel<TO, 1>), dim3(capped_grid((threads + 255) / 256, 8192)), dim3(256), 0, stream(),
                         ptr<TO>(out), o.data_ptr<float>(), tk.data_ptr<float>(), N, H, G, Dv);
  });
  HIP_CHECK_LAST();
  return out;
}

}  // namespace serving
}  // namespace cai
