// Normalisation kernels of the serving path (float32 statistics):
//   grouped_rms_norm   : per-group RMS scaling of a row, optional in-place add
//                        to the float32 residual stream;
//   head_rms_norm_gate : per-head RMS norm of [N, H, D] with a shared [D]
//                        weight and an optional sigmoid gate;
//   merge_rms_norm     : two branch rows, each full-width RMS-normed with its
//                        own weight, averaged, group-normed and added to the
//                        residual — one pass, the merged row staged in LDS;
//   add_rms_norm       : residual += a (+ b) in place and, when a weight is
//                        given, the RMS norm of the new residual row for the
//                        next pre-norm layer, in one launch;
//   gated_grouped_rms_norm : x * silu(gate), then the grouped RMS norm;
//   add_layer_norm     : centred norm (weight, no bias) of a sublayer's output
//                        added, scaled, to the residual in place, and the
//                        centred norm of the new residual row for the next
//                        sublayer, in one launch.
#include "serving_common.h"

namespace cai {
namespace serving {

// One wave per (row, group).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void grouped_rms_norm_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TI* __restrict__ x, long xs, const float* __restrict__ w,
    long units, int groups, int gs, float eps) {
  const int lane = threadIdx.x & 63;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= units) return;
  const long row = unit / groups;
  const int g = (int)(unit % groups);
  const long base = (row * groups + g) * (long)gs;   // in the dense output / residual
  const TI* xr = x + row * xs + (long)g * gs;        // the input's rows may be strided
  float ssq = 0.0f;
#pragma unroll 8
  for (int i = lane; i < gs; i += 64) {  // unrolled: the loads of a row are in flight together
    const float v = ldf(xr + i);
    ssq += v * v;
  }
  ssq = wave_reduce_sum(ssq);
  const float inv = 1.0f / sqrtf(ssq / (float)gs + eps);
#pragma unroll 8
  for (int i = lane; i < gs; i += 64) {
    const float y = ldf(xr + i) * inv * w[g * gs + i];
    if (residual != nullptr) residual[base + i] += y;
    else stf(out + base + i, y);
  }
}

at::Tensor grouped_rms_norm(at::Tensor x, at::Tensor weight, int64_t groups, double eps,
                            c10::optional<at::Tensor> residual, at::ScalarType out_dtype) {
  check_act(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1, "x must be [N, W] with unit inner stride");
  const long N = x.size(0);
  const int W = (int)x.size(1);
  const long xs = x.stride(0);
  TORCH_CHECK(groups > 0 && W % groups == 0);
  at::Tensor w = f32c(weight);
  TORCH_CHECK(w.numel() == W);
  float* res = nullptr;
  at::Tensor out;
  if (residual.has_value()) {
    TORCH_CHECK(is_f32(*residual) && residual->is_contiguous() && residual->sizes() == x.sizes() && x.is_contiguous(),
                "residual must be contiguous float32 of x's shape, and x contiguous with it");
    res = residual->data_ptr<float>();
    out = *residual;
  } else {
    out = at::empty({N, W}, x.options().dtype(out_dtype));
  }
  if (N == 0) return out;
  const long units = N * groups;
  const unsigned grid = (unsigned)((units + 3) / 4);
  SERVING_DISPATCH_ACT(x, TI, {
    if (res != nullptr) {
      hipLaunchKernelGGL((grouped_rms_norm_kernel<TI, float>), dim3(grid), dim3(256), 0, stream(), (float*)nullptr, res,
                         ptr<TI>(x), xs, w.data_ptr<float>(), units, (int)groups, W / (int)groups, (float)eps);
    } else {
      SERVING_DISPATCH_ACT(out, TO, {
        hipLaunchKernelGGL((grouped_rms_norm_kernel<TI, TO>), dim3(grid), dim3(256), 0, stream(), ptr<TO>(out),
                           (float*)nullptr, ptr<TI>(x), xs, w.data_ptr<float>(), units, (int)groups, W / (int)groups,
                           (float)eps);
      });
    }
  });
  HIP_CHECK_LAST();
  return out;
}

// One wave per (n, h). x row-strided: element (n, h, d) at n*xs + h*D + d.
template <typename TI, typename TG, typename TO>
__global__ __launch_bounds__(256) void head_rms_norm_gate_kernel(
    TO* __restrict__ out, const TI* __restrict__ x, long xs, const float* __restrict__ w, const TG* __restrict__ gate,
    long gs, long units, int H, int D, float eps) {
  const int lane = threadIdx.x & 63;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= units) return;
  const long n = unit / H;
  const int h = (int)(unit % H);
  const TI* xr = x + n * xs + (long)h * D;
  float ssq = 0.0f;
  for (int i = lane; i < D; i += 64) {
    const float v = ldf(xr + i);
    ssq += v * v;
  }
  ssq = wave_reduce_sum(ssq);
  const float inv = 1.0f / sqrtf(ssq / (float)D + eps);
  for (int i = lane; i < D; i += 64) {
    float y = ldf(xr + i) * inv * w[i];
    if (gate != nullptr) y *= sigmoidf_(ldf(gate + n * gs + (long)h * D + i));
    stf(out + (n * H + h) * (long)D + i, y);
  }
}

at::Tensor head_rms_norm_gate(at::Tensor x, at::Tensor weight, double eps, c10::optional<at::Tensor> gate,
                              at::ScalarType out_dtype) {
  check_act(x, "x");
  TORCH_CHECK(x.dim() == 3 && x.stride(2) == 1 && x.stride(1) == x.size(2), "x must be [N, H, D] with dense rows");
  const long N = x.size(0);
  const int H = (int)x.size(1), D = (int)x.size(2);
  at::Tensor w = f32c(weight);
  TORCH_CHECK(w.numel() == D);
  at::Tensor out = at::empty({N, H, D}, x.options().dtype(out_dtype));
  if (N == 0) return out;
  long gs = 0;
  if (gate.has_value()) {
    check_act(*gate, "gate");
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == N && gate->size(1) == (long)H * D && gate->stride(1) == 1);
    gs = gate->stride(0);
  }
  const long units = N * H;
  const unsigned grid = (unsigned)((units + 3) / 4);
  SERVING_DISPATCH_ACT(x, TI, {
    SERVING_DISPATCH_ACT(out, TO, {
      if (gate.has_value()) {
        SERVING_DISPATCH_ACT(*gate, TG, {
          hipLaunchKernelGGL((head_rms_norm_gate_kernel<TI, TG, TO>), dim3(grid), dim3(256), 0, stream(), ptr<TO>(out),
                             ptr<TI>(x), (long)x.stride(0), w.data_ptr<float>(), ptr<TG>(*gate), gs, units, H, D,
                             (float)eps);
        });
      } else {
        hipLaunchKernelGGL((head_rms_norm_gate_kernel<TI, float, TO>), dim3(grid), dim3(256), 0, stream(),
                           ptr<TO>(out), ptr<TI>(x), (long)x.stride(0), w.data_ptr<float>(), (const float*)nullptr,
                           0L, units, H, D, (float)eps);
      }
    });
  });
  HIP_CHECK_LAST();
  return out;
}

// One block per row; the merged row lives in LDS (W floats).
template <typename T>
__global__ __launch_bounds__(256) void merge_rms_norm_kernel(
    float* __restrict__ residual, const T* __restrict__ a, const float* __restrict__ wa, const T* __restrict__ b,
    const float* __restrict__ wb, const float* __restrict__ wo, int W, int groups, float eps) {
  extern __shared__ float merged[];
  __shared__ float red[8];
  const long row = blockIdx.x;
  const T* ar = a + row * W;
  const T* br = b + row * W;
  float sa = 0.0f, sb = 0.0f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float va = ldf(ar + i), vb = ldf(br + i);
    sa += va * va;
    sb += vb * vb;
  }
  sa = block_reduce_sum(sa, red);
  sb = block_reduce_sum(sb, red);
  const float ia = 1.0f / sqrtf(sa / (float)W + eps), ib = 1.0f / sqrtf(sb / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    merged[i] = 0.5f * (ldf(ar + i) * ia * wa[i] + ldf(br + i) * ib * wb[i]);
  __syncthreads();
  const int gs = W / groups, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  for (int g = threadIdx.x >> 6; g < groups; g += nw) {
    float s = 0.0f;
    for (int i = lane; i < gs; i += 64) {
      const float v = merged[g * gs + i];
      s += v * v;
    }
    s = wave_reduce_sum(s);
    const float inv = 1.0f / sqrtf(s / (float)gs + eps);
    for (int i = lane; i < gs; i += 64) residual[row * W + g * gs + i] += merged[g * gs + i] * inv * wo[g * gs + i];
  }
}

at::Tensor merge_rms_norm(at::Tensor a, at::Tensor wa, at::Tensor b, at::Tensor wb, double eps, at::Tensor out_w,
                          int64_t groups, at::Tensor residual) {
  check_act(a, "a");
  TORCH_CHECK(a.dim() == 2 && a.is_contiguous() && b.is_contiguous() && a.sizes() == b.sizes() &&
              a.scalar_type() == b.scalar_type());
  TORCH_CHECK(is_f32(residual) && residual.is_contiguous() && residual.sizes() == a.sizes());
  const long N = a.size(0);
  const int W = (int)a.size(1);
  TORCH_CHECK(groups > 0 && W % groups == 0 && W * 4 <= 64 * 1024, "row too wide for the LDS-staged merge");
  at::Tensor fa = f32c(wa), fb = f32c(wb), fo = f32c(out_w);
  TORCH_CHECK(fa.numel() == W && fb.numel() == W && fo.numel() == W);
  if (N == 0) return residual;
  SERVING_DISPATCH_ACT(a, T, {
    hipLaunchKernelGGL(merge_rms_norm_kernel<T>, dim3((unsigned)N), dim3(256), (size_t)W * 4, stream(),
                       residual.data_ptr<float>(), ptr<T>(a), fa.data_ptr<float>(), ptr<T>(b), fb.data_ptr<float>(),
                       fo.data_ptr<float>(), W, (int)groups, (float)eps);
  });
  HIP_CHECK_LAST();
  return residual;
}

// One block per row. Pass 1 forms r = residual + (a + b) in float32, stores it and sums r^2; pass 2
// (only with a weight) re-reads the elements this same thread stored and writes the normed row.
template <typename TA, typename TB, typename TO>
__global__ __launch_bounds__(256) void add_rms_norm_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TA* __restrict__ a, const TB* __restrict__ b,
    const float* __restrict__ w, int W, float eps) {
  __shared__ float red[8];
  const long row = blockIdx.x;
  float* rr = residual + row * W;
  float ssq = 0.0f;
#pragma unroll 4
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float add = ldf(a + row * W + i);
    if (b != nullptr) add += ldf(b + row * W + i);
    const float r = rr[i] + add;
    rr[i] = r;
    ssq += r * r;
  }
  if (w == nullptr) return;
  ssq = block_reduce_sum(ssq, red);
  const float inv = 1.0f / sqrtf(ssq / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + row * W + i, rr[i] * inv * w[i]);
}

// Row-in-registers form for rows of up to 2048 * CH elements (W a multiple of 8, 32-byte aligned
// operands): each thread owns CH chunks of 8 consecutive elements, reads every operand once with
// 16/32-byte loads, keeps the summed row in registers across the reduction and writes residual and
// normed row once.
template <typename TA, typename TB, typename TO, int CH>
__global__ __launch_bounds__(256) void add_rms_norm_rows_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TA* __restrict__ a, const TB* __restrict__ b,
    const float* __restrict__ w, int W, float eps) {
  __shared__ float red[8];
  const long row = blockIdx.x;
  float r[CH][8];
  float ssq = 0.0f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (threadIdx.x + 256 * c) * 8;
    if (i < W) {
      float av[8], bv[8];
      load8(residual + row * W + i, r[c]);
      load8(a + row * W + i, av);
      if (b != nullptr) load8(b + row * W + i, bv);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        r[c][e] += b != nullptr ? av[e] + bv[e] : av[e];
        ssq += r[c][e] * r[c][e];
      }
      store8(residual + row * W + i, r[c]);
    }
  }
  if (w == nullptr) return;
  ssq = block_reduce_sum(ssq, red);
  const float inv = 1.0f / sqrtf(ssq / (float)W + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (threadIdx.x + 256 * c) * 8;
    if (i < W) {
      float wv[8];
      load8(w + i, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[e] *= r[c][e] * inv;
      store8(out + row * W + i, wv);
    }
  }
}

c10::optional<at::Tensor> add_rms_norm(at::Tensor residual, at::Tensor a, c10::optional<at::Tensor> b,
                                       c10::optional<at::Tensor> weight, double eps, at::ScalarType out_dtype) {
  check_act(a, "a");
  TORCH_CHECK(residual.is_cuda() && is_f32(residual) && residual.dim() == 2 && residual.is_contiguous(),
              "residual must be contiguous float32 [N, W]");
  TORCH_CHECK(a.is_contiguous() && a.sizes() == residual.sizes(), "a must be contiguous and of the residual's shape");
  if (b.has_value()) {
    check_act(*b, "b");
    TORCH_CHECK(b->is_contiguous() && b->sizes() == residual.sizes(), "b must be contiguous and of the residual's shape");
  }
  const long N = residual.size(0);
  const int W = (int)residual.size(1);
  at::Tensor w, out;
  const float* wp = nullptr;
  if (weight.has_value()) {
    w = f32c(*weight);
    TORCH_CHECK(w.numel() == W);
    wp = w.data_ptr<float>();
    out = at::empty({N, W}, residual.options().dtype(out_dtype));
    check_act(out, "out");
  }
  if (N > 0) {
    // without a weight nothing is written through `out`: any instantiation of TO will do
    const at::Tensor& like = weight.has_value() ? out : residual;
    auto al32 = [](const at::Tensor& t) { return reinterpret_cast<uintptr_t>(t.data_ptr()) % 32 == 0; };
    const bool rows = W % 8 == 0 && W <= 2048 * 4 && al32(residual) && al32(a) && (!b.has_value() || al32(*b)) &&
                      (!weight.has_value() || (al32(out) && al32(w)));
    const float* nob = nullptr;
#define ADD_NORM_LAUNCH(TB_, bp)                                                                                        \
  do {                                                                                                                  \
    if (rows && W <= 2048)                                                                                              \
      hipLaunchKernelGGL((add_rms_norm_rows_kernel<TA, TB_, TO, 1>), dim3((unsigned)N), dim3(256), 0, stream(), op,    \
                         residual.data_ptr<float>(), ptr<TA>(a), bp, wp, W, (float)eps);                                \
    else if (rows && W <= 4096)                                                                                         \
      hipLaunchKernelGGL((add_rms_norm_rows_kernel<TA, TB_, TO, 2>), dim3((unsigned)N), dim3(256), 0, stream(), op,    \
                         residual.data_ptr<float>(), ptr<TA>(a), bp, wp, W, (float)eps);                                \
    else if (rows)                                                                                                      \
      hipLaunchKernelGGL((add_rms_norm_rows_kernel<TA, TB_, TO, 4>), dim3((unsigned)N), dim3(256), 0, stream(), op,    \
                         residual.data_ptr<float>(), ptr<TA>(a), bp, wp, W, (float)eps);                                \
    else                                                                                                                \
      hipLaunchKernelGGL((add_rms_norm_kernel<TA, TB_, TO>), dim3((unsigned)N), dim3(256), 0, stream(), op,            \
                         residual.data_ptr<float>(), ptr<TA>(a), bp, wp, W, (float)eps);                                \
  } while (0)
    SERVING_DISPATCH_ACT(a, TA, {
      SERVING_DISPATCH_ACT(like, TO, {
        TO* op = weight.has_value() ? ptr<TO>(out) : (TO*)nullptr;
        if (b.has_value()) {
          SERVING_DISPATCH_ACT(*b, TB, { ADD_NORM_LAUNCH(TB, ptr<TB>(*b)); });
        } else {
          ADD_NORM_LAUNCH(float, nob);
        }
      });
    });
#undef ADD_NORM_LAUNCH
    HIP_CHECK_LAST();
  }
  if (!weight.has_value()) return c10::nullopt;
  return out;
}

// ------------------------------------------------------- gate, then grouped RMS norm
// One wave per (row, group): out = rms_unit(x * silu(gate)) * w over the group. x dense [N, W]
// (float32 or an activation type), gate row-strided.
template <typename TX, typename TG, typename TO>
__global__ __launch_bounds__(256) void gated_grouped_rms_norm_kernel(
    TO* __restrict__ out, const TX* __restrict__ x, const TG* __restrict__ gate, long gstride,
    const float* __restrict__ w, long units, int groups, int gs, float eps) {
  const int lane = threadIdx.x & 63;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= units) return;
  const long row = unit / groups;
  const int g = (int)(unit % groups);
  const long base = (row * groups + g) * (long)gs;
  const TG* gr = gate + row * gstride + (long)g * gs;
  float ssq = 0.0f;
#pragma unroll 4
  for (int i = lane; i < gs; i += 64) {
    const float z = ldf(gr + i);
    const float v = ldf(x + base + i) * (z * sigmoidf_(z));
    ssq += v * v;
  }
  ssq = wave_reduce_sum(ssq);
  const float inv = 1.0f / sqrtf(ssq / (float)gs + eps);
#pragma unroll 4
  for (int i = lane; i < gs; i += 64) {
    const float z = ldf(gr + i);
    stf(out + base + i, ldf(x + base + i) * (z * sigmoidf_(z)) * inv * w[g * gs + i]);
  }
}

at::Tensor gated_grouped_rms_norm(at::Tensor x, at::Tensor gate, at::Tensor weight, int64_t groups, double eps,
                                  at::ScalarType out_dtype) {
  check_act(x, "x"); check_act(gate, "gate");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "x must be contiguous [N, W]");
  TORCH_CHECK(gate.dim() == 2 && gate.sizes() == x.sizes() && gate.stride(1) == 1, "gate must be [N, W] with unit inner stride");
  const long N = x.size(0);
  const int W = (int)x.size(1);
  TORCH_CHECK(groups > 0 && W % groups == 0);
  at::Tensor w = f32c(weight);
  TORCH_CHECK(w.numel() == W);
  at::Tensor out = at::empty({N, W}, x.options().dtype(out_dtype));
  check_act(out, "out");
  if (N == 0) return out;
  const long units = N * groups;
  const unsigned grid = (unsigned)((units + 3) / 4);
  SERVING_DISPATCH_ACT(x, TX, {
    SERVING_DISPATCH_ACT(gate, TG, {
      SERVING_DISPATCH_ACT(out, TO, {
        hipLaunchKernelGGL((gated_grouped_rms_norm_kernel<TX, TG, TO>), dim3(grid), dim3(256), 0, stream(), ptr<TO>(out),
                           ptr<TX>(x), ptr<TG>(gate), (long)gate.stride(0), w.data_ptr<float>(), units, (int)groups,
                           W / (int)groups, (float)eps);
      });
    });
  });
  HIP_CHECK_LAST();
  return out;
}

// ------------------------------------------------- centred norm on the way in and out
// One block per row. With a residual: residual += mult * layer_norm(y) * w_out in place; then, with
// w_next, out = layer_norm(residual) * w_next. Without a residual: out = layer_norm(y) * w_next.
// layer_norm(v) = (v - mean) / sqrt(mean((v - mean)^2) + eps): the variance is taken from the
// deviations (a second pass over registers), not from the mean of squares.
// CH > 0: each thread owns CH chunks of 8 consecutive elements in registers (W a multiple of 8 up to
// 2048 * CH, aligned operands), every operand is read once with 16/32-byte loads. CH == 0: any W,
// the row is staged in LDS.
template <typename TY, typename TO, int CH>
__global__ __launch_bounds__(256) void add_layer_norm_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TY* __restrict__ y, const float* __restrict__ w_out,
    float mult, const float* __restrict__ w_next, int W, float eps) {
  __shared__ float red[8];
  extern __shared__ __align__(16) float rowbuf[];
  const long row = blockIdx.x;
  const float invW = 1.0f / (float)W;
  if constexpr (CH > 0) {
    float r[CH][8];
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int i = (threadIdx.x + 256 * c) * 8;
      if (i < W) {
        load8(y + row * W + i, r[c]);
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += r[c][e];
      }
    }
    if (residual != nullptr) {
      const float mean = block_reduce_sum(sum, red) * invW;
      float ssq = 0.0f;
#pragma unroll
      for (int c = 0; c < CH; ++c)
        if ((threadIdx.x + 256 * c) * 8 < W) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            r[c][e] -= mean;
            ssq += r[c][e] * r[c][e];
          }
        }
      const float inv = mult / sqrtf(block_reduce_sum(ssq, red) * invW + eps);
      sum = 0.0f;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int i = (threadIdx.x + 256 * c) * 8;
        if (i < W) {
          float wv[8], xv[8];
          load8(w_out + i, wv);
          load8(residual + row * W + i, xv);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            r[c][e] = xv[e] + r[c][e] * inv * wv[e];
            sum += r[c][e];
          }
          store8(residual + row * W + i, r[c]);
        }
      }
      if (w_next == nullptr) return;
    }
    const float mean = block_reduce_sum(sum, red) * invW;
    float ssq = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c)
      if ((threadIdx.x + 256 * c) * 8 < W) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          r[c][e] -= mean;
          ssq += r[c][e] * r[c][e];
        }
      }
    const float inv = 1.0f / sqrtf(block_reduce_sum(ssq, red) * invW + eps);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int i = (threadIdx.x + 256 * c) * 8;
      if (i < W) {
        float wv[8];
        load8(w_next + i, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) wv[e] *= r[c][e] * inv;
        store8(out + row * W + i, wv);
      }
    }
  } else {
    float sum = 0.0f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float v = ldf(y + row * W + i);
      rowbuf[i] = v;
      sum += v;
    }
    if (residual != nullptr) {
      const float mean = block_reduce_sum(sum, red) * invW;
      float ssq = 0.0f;
      for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float d = rowbuf[i] - mean;
        ssq += d * d;
      }
      const float inv = mult / sqrtf(block_reduce_sum(ssq, red) * invW + eps);
      sum = 0.0f;
      for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float v = residual[row * W + i] + (rowbuf[i] - mean) * inv * w_out[i];
        residual[row * W + i] = v;
        rowbuf[i] = v;
        sum += v;
      }
      if (w_next == nullptr) return;
    }
    const float mean = block_reduce_sum(sum, red) * invW;
    float ssq = 0.0f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float d = rowbuf[i] - mean;
      ssq += d * d;
    }
    const float inv = 1.0f / sqrtf(block_reduce_sum(ssq, red) * invW + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + row * W + i, (rowbuf[i] - mean) * inv * w_next[i]);
  }
}

c10::optional<at::Tensor> add_layer_norm(c10::optional<at::Tensor> residual, at::Tensor y,
                                         c10::optional<at::Tensor> w_out, double mult,
                                         c10::optional<at::Tensor> w_next, double eps, at::ScalarType out_dtype) {
  check_act(y, "y");
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous(), "y must be contiguous [N, W]");
  const long N = y.size(0);
  const int W = (int)y.size(1);
  TORCH_CHECK(residual.has_value() == w_out.has_value(), "a residual needs the weight of the norm on its way in");
  TORCH_CHECK(residual.has_value() || w_next.has_value(), "nothing to compute");
  float* rp = nullptr;
  at::Tensor wo, wn, out;
  const float *wop = nullptr, *wnp = nullptr;
  if (residual.has_value()) {
    TORCH_CHECK(residual->is_cuda() && is_f32(*residual) && residual->is_contiguous() && residual->sizes() == y.sizes(),
                "residual must be contiguous float32 of y's shape");
    rp = residual->data_ptr<float>();
    wo = f32c(*w_out);
    TORCH_CHECK(wo.numel() == W);
    wop = wo.data_ptr<float>();
  }
  if (w_next.has_value()) {
    wn = f32c(*w_next);
    TORCH_CHECK(wn.numel() == W);
    wnp = wn.data_ptr<float>();
    out = at::empty({N, W}, y.options().dtype(out_dtype));
    check_act(out, "out");
  }
  if (N > 0) {
    const at::Tensor& like = w_next.has_value() ? out : y;   // without w_next nothing is written through `out`
    auto al32 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 32 == 0; };
    const bool rows = W % 8 == 0 && W <= 2048 * 4 && al32(y.data_ptr()) && (rp == nullptr || (al32(rp) && al32(wop))) &&
                      (wnp == nullptr || (al32(wnp) && al32(out.data_ptr())));
    TORCH_CHECK(rows || (size_t)W * sizeof(float) <= 64 * 1024, "row too long for the norm kernel");
#define LN_LAUNCH(CH_, SMEM_)                                                                                      \
  hipLaunchKernelGGL((add_layer_norm_kernel<TY, TO, CH_>), dim3((unsigned)N), dim3(256), SMEM_, stream(), op, rp, \
                     ptr<TY>(y), wop, (float)mult, wnp, W, (float)eps)
    SERVING_DISPATCH_ACT(y, TY, {
      SERVING_DISPATCH_ACT(like, TO, {
        TO* op = w_next.has_value() ? ptr<TO>(out) : (TO*)nullptr;
        if (rows && W <= 2048) LN_LAUNCH(1, 0);
        else if (rows && W <= 4096) LN_LAUNCH(2, 0);
        else if (rows) LN_LAUNCH(4, 0);
        else LN_LAUNCH(0, (size_t)W * sizeof(float));
      });
    });
#undef LN_LAUNCH
    HIP_CHECK_LAST();
  }
  if (!w_next.has_value()) return c10::nullopt;
  return out;
}

// ------------------------------------------- norm on a sublayer's output, one number as weight
// One block per row: y = sa * a (+ sb * b); residual += gain * y / sqrt(mean(y^2) + eps) (float32,
// in place); with `cast` the updated row is also stored in an activation type — the next
// sublayer's input when sublayers read the stream itself. The row's y stays in registers
// (W <= 256 * PER) between the reduction and the update.
template <typename TA, typename TB, typename TO, int PER>
__global__ __launch_bounds__(256) void add_scaled_unit_norm_kernel(
    TO* __restrict__ cast, float* __restrict__ residual, const TA* __restrict__ a, const TB* __restrict__ b, float sa,
    float sb, float gain, int W, float eps) {
  __shared__ float red[8];
  const long row = blockIdx.x;
  float y[PER];
  float ssq = 0.0f;
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int i = threadIdx.x + 256 * r;
    y[r] = 0.0f;
    if (i < W) {
      y[r] = sa * ldf(a + row * W + i);
      if (b != nullptr) y[r] += sb * ldf(b + row * W + i);
      ssq += y[r] * y[r];
    }
  }
  ssq = block_reduce_sum(ssq, red);
  const float f = gain / sqrtf(ssq / (float)W + eps);
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int i = threadIdx.x + 256 * r;
    if (i < W) {
      const float v = residual[row * W + i] + f * y[r];
      residual[row * W + i] = v;
      if (cast != nullptr) stf(cast + row * W + i, v);
    }
  }
}

c10::optional<at::Tensor> add_scaled_unit_norm(at::Tensor residual, at::Tensor a, c10::optional<at::Tensor> b,
                                               double scale_a, double scale_b, double gain, double eps,
                                               c10::optional<at::ScalarType> out_dtype) {
  TORCH_CHECK(residual.is_cuda() && is_f32(residual) && residual.dim() == 2 && residual.is_contiguous(),
              "residual must be contiguous float32 [N, W]");
  check_act(a, "a");
  TORCH_CHECK(a.is_contiguous() && a.sizes() == residual.sizes(), "a must be contiguous and of the residual's shape");
  if (b.has_value()) {
    check_act(*b, "b");
    TORCH_CHECK(b->is_contiguous() && b->sizes() == residual.sizes(), "b must be contiguous and of the residual's shape");
  }
  const long N = residual.size(0);
  const int W = (int)residual.size(1);
  TORCH_CHECK(W <= 256 * 64, "rows of up to 16384 elements");
  at::Tensor out;
  if (out_dtype.has_value()) {
    TORCH_CHECK(*out_dtype == at::kFloat || *out_dtype == at::kBFloat16);
    out = at::empty({N, W}, residual.options().dtype(*out_dtype));
  }
  if (N > 0) {
    const at::Tensor like = out_dtype.has_value() ? out : residual;
    const float* nob = nullptr;
#define ASUN_LAUNCH(TB_, BP_, PER_)                                                                                     \
  hipLaunchKernelGGL((add_scaled_unit_norm_kernel<TA, TB_, TO, PER_>), dim3((unsigned)N), dim3(256), 0, stream(), op,   \
                     residual.data_ptr<float>(), ptr<TA>(a), BP_, (float)scale_a, (float)scale_b, (float)gain, W,       \
                     (float)eps)
#define ASUN_SIZES(TB_, BP_)                     \
  do {                                           \
    if (W <= 1024) ASUN_LAUNCH(TB_, BP_, 4);     \
    else if (W <= 4096) ASUN_LAUNCH(TB_, BP_, 16); \
    else ASUN_LAUNCH(TB_, BP_, 64);              \
  } while (0)
    SERVING_DISPATCH_ACT(a, TA, {
      SERVING_DISPATCH_ACT(like, TO, {
        TO* op = out_dtype.has_value() ? ptr<TO>(out) : (TO*)nullptr;
        if (b.has_value()) {
          SERVING_DISPATCH_ACT(*b, TB, { ASUN_SIZES(TB, ptr<TB>(*b)); });
        } else {
          ASUN_SIZES(float, nob);
        }
      });
    });
#undef ASUN_SIZES
#undef ASUN_LAUNCH
    HIP_CHECK_LAST();
  }
  if (!out_dtype.has_value()) return c10::nullopt;
  return out;
}

}  // namespace serving
}  // namespace cai
