// RMSNorm over the last dimension, one workgroup per row, with three optional
// fusions that each save one pass over the activations:
//   * residual add:  r = round(x + r) is written back, then the norm is taken
//     of the rounded r (the value the next layer will also read);
//   * row gather:    only the listed rows of x are normed (final norm before
//     the LM head);
//   * weight offset: y = x * inv * (w + offset), offset 0 for plain gains and
//     1 for gains stored around zero.
// ss, inv and all products are float; one rounding on store.
//
// Reference behaviour: crates/kernels/cuda/norm.cu:41-116,192-221 and
// rmsnorm_core.cuh:63-81 (inv = 1/sqrt(ss/n + eps), weight multiplies
// directly), norm.cu:69-85 (the add is rounded before it is normed).
#include "common.cuh"

using namespace dinfer;

namespace {

template <class S>
__global__ void __launch_bounds__(256) rmsnorm_kernel(const S* __restrict__ x, S* __restrict__ residual,
                                                      const int32_t* __restrict__ rows, const void* __restrict__ w,
                                                      int wf32, S* __restrict__ out, int64_t width, int64_t ld_x,
                                                      int64_t ld_res, float eps, float w_offset) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : r;
  const S* xr = x + src * ld_x;
  S* rr = residual ? residual + src * ld_res : nullptr;
  S* o = out + r * width;
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    float v = to_f32(xr[i]);
    if (rr) {
      const S s = from_f32<S>(v + to_f32(rr[i]));
      rr[i] = s;
      v = to_f32(s);
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  const S* src2 = rr ? rr : xr;  // each thread re-reads only what it wrote itself
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x)
    o[i] = from_f32<S>(to_f32(src2[i]) * inv * (ld_param<S>(w, i, wf32) + w_offset));
}

// bf16 rows whose width is a multiple of 8 and at most 256*8*ITERS: each
// thread keeps its 8-element pieces in registers between the two phases.
template <int ITERS>
__global__ void __launch_bounds__(256) rmsnorm_bf16x8_kernel(const bf16* __restrict__ x, bf16* __restrict__ residual,
                                                             const int32_t* __restrict__ rows,
                                                             const void* __restrict__ w, int wf32,
                                                             bf16* __restrict__ out, int64_t width, int64_t ld_x,
                                                             int64_t ld_res, float eps, float w_offset) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : r;
  const bf16x8* xr = (const bf16x8*)(x + src * ld_x);
  bf16x8* rr = residual ? (bf16x8*)(residual + src * ld_res) : nullptr;
  bf16x8* o = (bf16x8*)(out + r * width);
  const int n8 = (int)(width / 8);
  float v[ITERS][8];
  float g[ITERS][8];  // the gains: loaded with the row, not after the sum (one memory round trip less)
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
      const bf16x8 xv = xr[i];
      if (wf32) {
        const float* wp = (const float*)w + (int64_t)i * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) g[it][j] = wp[j] + w_offset;
      } else {
        const bf16x8 wv = ((const bf16x8*)w)[i];
#pragma unroll
        for (int j = 0; j < 8; ++j) g[it][j] = (float)wv[j] + w_offset;
      }
      if (rr) {
        const bf16x8 rv = rr[i];
        bf16x8 s;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          s[j] = (bf16)((float)xv[j] + (float)rv[j]);
          v[it][j] = (float)s[j];
        }
        rr[i] = s;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[it][j] = (float)xv[j];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[it][j] * v[it][j];
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
      bf16x8 y;
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = (bf16)(v[it][j] * inv * g[it][j]);
      o[i] = y;
    }
  }
}

// Layer norm with gain and bias over the last dimension: y = (x - mean) / sqrt(var + eps) * w + b, var the mean of the
// squared deviations (two passes over the row, which waits in LDS in float). The operands may differ in storage: the
// residual stream may be float where the branch added to it and the normed row are bf16. With a residual,
// r = round(x + r) is written back in the residual's own type first and normed as stored.
__device__ __forceinline__ float ld_any(const void* p, int64_t i, int dt) {
  return dt == DT_F32 ? ((const float*)p)[i] : (float)((const bf16*)p)[i];
}
__device__ __forceinline__ void st_any(void* p, int64_t i, int dt, float v) {
  if (dt == DT_F32) ((float*)p)[i] = v; else ((bf16*)p)[i] = (bf16)v;
}
__device__ __forceinline__ float round_any(float v, int dt) { return dt == DT_F32 ? v : (float)(bf16)v; }

__global__ void __launch_bounds__(256) layernorm_kernel(const void* __restrict__ x, int x_dt, void* __restrict__ residual,
                                                        int r_dt, const int32_t* __restrict__ rows,
                                                        const void* __restrict__ w, const void* __restrict__ b, int p_dt,
                                                        void* __restrict__ out, int o_dt, int64_t width, int64_t ld_x,
                                                        int64_t ld_res, float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : r;
  float sum = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    float v = ld_any(x, src * ld_x + i, x_dt);
    if (residual) {
      v = round_any(v + ld_any(residual, src * ld_res + i, r_dt), r_dt);
      st_any(residual, src * ld_res + i, r_dt, v);
    }
    row[i] = v;
    sum += v;
  }
  const float mean = block_sum(sum, red) / (float)width;
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {   // each thread re-reads what it wrote itself
    const float d = row[i] - mean;
    ss = add_square(ss, d);
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    const float y = (row[i] - mean) * inv * ld_any(w, i, p_dt) + (b ? ld_any(b, i, p_dt) : 0.f);
    st_any(out, r * width + i, o_dt, y);
  }
}

// The same for widths that are multiples of 8 up to 256 * 8 * ITERS: a thread keeps its 8-entry pieces in registers
// between the passes (one read of the row, no LDS but for the two sums), and moves them 16 or 32 bytes at a time.
template <class SX, class SR, class SO, int ITERS>
__global__ void __launch_bounds__(256) layernorm_regs_kernel(const SX* __restrict__ x, SR* __restrict__ residual,
                                                             const int32_t* __restrict__ rows,
                                                             const float* __restrict__ w, const float* __restrict__ b,
                                                             SO* __restrict__ out, int64_t width, int64_t ld_x,
                                                             int64_t ld_res, float eps) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : r;
  const SX* xr = x + src * ld_x;
  SR* rr = residual ? residual + src * ld_res : nullptr;
  const int n8 = (int)(width / 8);
  float v[ITERS][8];
  float sum = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[it][j] = to_f32(xr[(int64_t)i * 8 + j]);
      if (rr) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const SR s = from_f32<SR>(v[it][j] + to_f32(rr[(int64_t)i * 8 + j]));
          rr[(int64_t)i * 8 + j] = s;
          v[it][j] = to_f32(s);
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) sum += v[it][j];
    }
  }
  const float mean = block_sum(sum, red) / (float)width;
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = add_square(ss, v[it][j] - mean);
    }
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
  SO* o = out + r * width;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int64_t c = (int64_t)i * 8 + j;
        o[c] = from_f32<SO>((v[it][j] - mean) * inv * w[c] + (b ? b[c] : 0.f));
      }
    }
  }
}

template <class SX, class SR, class SO>
void launch_layernorm_regs(const void* x, void* residual, const int32_t* rows, const void* w, const void* b, void* out,
                           int64_t n_rows, int64_t width, int64_t ld_x, int64_t ld_res, float eps, hipStream_t stream) {
  const unsigned g = (unsigned)n_rows;
#define LN(IT)                                                                                                        \
  layernorm_regs_kernel<SX, SR, SO, IT><<<g, 256, 0, stream>>>((const SX*)x, (SR*)residual, rows, (const float*)w,    \
                                                               (const float*)b, (SO*)out, width, ld_x, ld_res, eps)
  if (width <= 256 * 8) LN(1);
  else if (width <= 256 * 8 * 2) LN(2);
  else LN(4);
#undef LN
}

inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

}  // namespace

// x [*, width] with row stride ld_x; residual (may be null) has row stride
// ld_res and is updated in place; rows (may be null) lists the n_rows source
// rows; out is dense [n_rows, width]. w has `width` elements, float if w_f32.
extern "C" int dinfer_rmsnorm(int dtype, const void* x, void* residual, const int32_t* rows, const void* w, int w_f32,
                              void* out, int64_t n_rows, int64_t width, int64_t ld_x, int64_t ld_res, float eps,
                              float w_offset, hipStream_t stream) {
  if (n_rows <= 0) return OK;
  if (width <= 0 || ld_x < width || (residual && ld_res < width) || n_rows > 0x7fffffff) return ERR_BAD_SHAPE;
  if (dtype == DT_BF16) {
    const bool vec = width % 8 == 0 && ld_x % 8 == 0 && (!residual || ld_res % 8 == 0) && aligned16(x) &&
                     aligned16(out) && aligned16(w) && (!residual || aligned16(residual)) && width <= 256 * 8 * 4;
    const bf16* xp = (const bf16*)x;
    bf16* rp = (bf16*)residual;
    bf16* op = (bf16*)out;
    if (vec && width <= 256 * 8) {
      rmsnorm_bf16x8_kernel<1><<<(unsigned)n_rows, 256, 0, stream>>>(xp, rp, rows, w, w_f32, op, width, ld_x, ld_res,
                                                                     eps, w_offset);
    } else if (vec && width <= 256 * 8 * 2) {
      rmsnorm_bf16x8_kernel<2><<<(unsigned)n_rows, 256, 0, stream>>>(xp, rp, rows, w, w_f32, op, width, ld_x, ld_res,
                                                                     eps, w_offset);
    } else if (vec) {
      rmsnorm_bf16x8_kernel<4><<<(unsigned)n_rows, 256, 0, stream>>>(xp, rp, rows, w, w_f32, op, width, ld_x, ld_res,
                                                                     eps, w_offset);
    } else {
      rmsnorm_kernel<bf16><<<(unsigned)n_rows, 256, 0, stream>>>(xp, rp, rows, w, w_f32, op, width, ld_x, ld_res, eps,
                                                                 w_offset);
    }
  } else if (dtype == DT_F32) {
    rmsnorm_kernel<float><<<(unsigned)n_rows, 256, 0, stream>>>((const float*)x, (float*)residual, rows, w, 1,
                                                                (float*)out, width, ld_x, ld_res, eps, w_offset);
  } else {
    return ERR_BAD_DTYPE;
  }
  return launch_status();
}

// x, residual (may be null), w and b (b may be null) and out each with a dtype code of their own (w and b share one).
// out is dense [n_rows, width]. Width up to 16,384 (the row waits in LDS).
extern "C" int dinfer_layernorm(const void* x, int x_dtype, void* residual, int res_dtype, const int32_t* rows,
                                const void* w, const void* b, int param_dtype, void* out, int out_dtype, int64_t n_rows,
                                int64_t width, int64_t ld_x, int64_t ld_res, float eps, hipStream_t stream) {
  if (n_rows <= 0) return OK;
  if (width <= 0 || ld_x < width || (residual && ld_res < width) || n_rows > 0x7fffffff) return ERR_BAD_SHAPE;
  for (int dt : {x_dtype, res_dtype, param_dtype, out_dtype})
    if (dt != DT_F32 && dt != DT_BF16) return ERR_BAD_DTYPE;
  // the combinations the engine meets, with float parameters, rows in registers: a float stream normed into the
  // engine's type, alone or after a branch of the engine's type was added to it
  if (param_dtype == DT_F32 && width % 8 == 0 && width <= 256 * 8 * 4 && ld_x % 8 == 0 && (!residual || ld_res % 8 == 0)) {
    const bool res_f32 = !residual || res_dtype == DT_F32;
    if (x_dtype == DT_F32 && res_f32 && out_dtype == DT_BF16) {
      launch_layernorm_regs<float, float, bf16>(x, residual, rows, w, b, out, n_rows, width, ld_x, ld_res, eps, stream);
      return launch_status();
    }
    if (x_dtype == DT_BF16 && res_f32 && out_dtype == DT_BF16) {
      launch_layernorm_regs<bf16, float, bf16>(x, residual, rows, w, b, out, n_rows, width, ld_x, ld_res, eps, stream);
      return launch_status();
    }
    if (x_dtype == DT_F32 && res_f32 && out_dtype == DT_F32) {
      launch_layernorm_regs<float, float, float>(x, residual, rows, w, b, out, n_rows, width, ld_x, ld_res, eps, stream);
      return launch_status();
    }
  }
  if (width > 16384) return ERR_UNSUPPORTED;
  layernorm_kernel<<<(unsigned)n_rows, 256, (size_t)width * sizeof(float), stream>>>(
      x, x_dtype, residual, res_dtype, rows, w, b, param_dtype, out, out_dtype, width, ld_x, ld_res, eps);
  return launch_status();
}

// A residual stream between norms on both sides of every sublayer:
//   stream[s] += mult * branch[s] / sqrt(mean(branch[s]^2) + eps_b) * (wb + off_b)       (with a branch)
//   out[r]     = stream[s] / sqrt(mean(stream[s]^2) + eps) * (w + off)                   (with an out)
// s = rows[r] where rows are given (the model's last norm, on the rows whose logits are wanted), else r. Branch,
// stream, gains and out each have a storage type of their own (a float stream beside bf16 branches and outputs);
// sums, divisions and the addition are float, each stored value is rounded once. The row waits in LDS.
namespace {

__global__ void __launch_bounds__(256) rmsnorm_stream_kernel(const void* __restrict__ branch, int b_dt, int64_t ld_b,
                                                             const void* __restrict__ wb, float eps_b, float off_b,
                                                             float mult, void* __restrict__ stream, int s_dt,
                                                             int64_t ld_s, const int32_t* __restrict__ rows,
                                                             const void* __restrict__ w, int p_dt,
                                                             void* __restrict__ out, int o_dt, float eps, float off,
                                                             int64_t width) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t s = rows ? (int64_t)rows[r] : r;
  float ss = 0.f;
  if (branch) {
    for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
      const float v = ld_any(branch, s * ld_b + i, b_dt);
      row[i] = v;
      ss = add_square(ss, v);
    }
    const float inv_b = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps_b);
    ss = 0.f;
    for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {   // each thread re-reads what it wrote itself
      const float y = row[i] * inv_b * (ld_any(wb, i, p_dt) + off_b);
      const float x = round_any(__builtin_fmaf(mult, y, ld_any(stream, s * ld_s + i, s_dt)), s_dt);
      st_any(stream, s * ld_s + i, s_dt, x);
      row[i] = x;
      ss = add_square(ss, x);
    }
  } else {
    for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
      const float x = ld_any(stream, s * ld_s + i, s_dt);
      row[i] = x;
      ss = add_square(ss, x);
    }
  }
  if (!out) return;
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x)
    st_any(out, r * width + i, o_dt, row[i] * inv * (ld_any(w, i, p_dt) + off));
}

// The same for the combination the engine meets (float stream, float gains, branch and out of one type), widths that
// are multiples of 8 up to 256 * 8 * ITERS: a thread keeps its 8-entry pieces in registers from the first read to the
// last store and moves them 16 or 32 bytes at a time; the gains are asked for with the row, not after the sums.
template <class SB, int ITERS>
__global__ void __launch_bounds__(256) rmsnorm_stream_regs_kernel(const SB* __restrict__ branch, int64_t ld_b,
                                                                  const float* __restrict__ wb, float eps_b, float off_b,
                                                                  float mult, float* __restrict__ stream, int64_t ld_s,
                                                                  const int32_t* __restrict__ rows,
                                                                  const float* __restrict__ w, SB* __restrict__ out,
                                                                  float eps, float off, int64_t width) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t s = rows ? (int64_t)rows[r] : r;
  const int n8 = (int)(width / 8);
  float x[ITERS][8], g[ITERS][8], y[ITERS][8];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
      const int64_t c = (int64_t)i * 8;
      const f32x4 s0 = *(const f32x4*)(stream + s * ld_s + c), s1 = *(const f32x4*)(stream + s * ld_s + c + 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[it][j] = s0[j];
        x[it][4 + j] = s1[j];
      }
      if (out) {
        const f32x4 g0 = *(const f32x4*)(w + c), g1 = *(const f32x4*)(w + c + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          g[it][j] = g0[j] + off;
          g[it][4 + j] = g1[j] + off;
        }
      }
      if (branch) {
        const f32x4 b0 = *(const f32x4*)(wb + c), b1 = *(const f32x4*)(wb + c + 4);
        float bv[8];
        if constexpr (sizeof(SB) == 2) {
          const bf16x8 p = *(const bf16x8*)(branch + s * ld_b + c);
#pragma unroll
          for (int j = 0; j < 8; ++j) bv[j] = (float)p[j];
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) bv[j] = to_f32(branch[s * ld_b + c + j]);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float v = bv[j];
          y[it][j] = v * ((j < 4 ? b0[j] : b1[j - 4]) + off_b);
          ss = add_square(ss, v);
        }
      }
    }
  }
  if (branch) {
    const float inv_b = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps_b);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int i = it * 256 + threadIdx.x;
      if (i < n8) {
        const int64_t c = (int64_t)i * 8;
        f32x4 s0, s1;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          x[it][j] = __builtin_fmaf(mult, y[it][j] * inv_b, x[it][j]);
          if (j < 4) s0[j] = x[it][j]; else s1[j - 4] = x[it][j];
        }
        *(f32x4*)(stream + s * ld_s + c) = s0;
        *(f32x4*)(stream + s * ld_s + c + 4) = s1;
      }
    }
  }
  if (!out) return;
  ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = add_square(ss, x[it][j]);
    }
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
      SB* o = out + r * width + (int64_t)i * 8;
      if constexpr (sizeof(SB) == 2) {
        bf16x8 p;
#pragma unroll
        for (int j = 0; j < 8; ++j) p[j] = (bf16)(x[it][j] * inv * g[it][j]);
        *(bf16x8*)o = p;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = from_f32<SB>(x[it][j] * inv * g[it][j]);
      }
    }
  }
}

template <class SB>
void launch_stream_regs(const void* branch, int64_t ld_b, const void* wb, float eps_b, float off_b, float mult, void* stream_,
                        int64_t ld_s, const int32_t* rows, const void* w, void* out, float eps, float off, int64_t n_rows,
                        int64_t width, hipStream_t stream) {
#define SN(IT)                                                                                                       \
  rmsnorm_stream_regs_kernel<SB, IT><<<(unsigned)n_rows, 256, 0, stream>>>(                                          \
      (const SB*)branch, ld_b, (const float*)wb, eps_b, off_b, mult, (float*)stream_, ld_s, rows, (const float*)w, \
      (SB*)out, eps, off, width)
  if (width <= 256 * 8) SN(1);
  else if (width <= 256 * 8 * 2) SN(2);
  else SN(4);
#undef SN
}

}  // namespace

// branch (may be null) [*, ld_b]; stream [*, ld_s], updated in place where a branch is given; out (may be null) dense
// [n_rows, width]; wb and w share the storage type param_dtype. Width up to 16,384.
extern "C" int dinfer_rmsnorm_stream(const void* branch, int branch_dtype, int64_t ld_b, const void* wb, float eps_b,
                                     float off_b, float mult, void* stream_, int stream_dtype, int64_t ld_s,
                                     const int32_t* rows, const void* w, int param_dtype, void* out, int out_dtype,
                                     float eps, float off, int64_t n_rows, int64_t width, hipStream_t stream) {
  if (n_rows <= 0) return OK;
  if (width <= 0 || ld_s < width || (branch && (ld_b < width || !wb)) || (out && !w) || (!branch && !out) ||
      n_rows > 0x7fffffff)
    return ERR_BAD_SHAPE;
  for (int dt : {branch_dtype, stream_dtype, param_dtype, out_dtype})
    if (dt != DT_F32 && dt != DT_BF16) return ERR_BAD_DTYPE;
  // a float stream with float gains, branch and out of one type, rows of whole 16-byte pieces: rows in registers
  const int io_dtype = branch ? branch_dtype : out_dtype;
  if (stream_dtype == DT_F32 && param_dtype == DT_F32 && (!branch || !out || branch_dtype == out_dtype) &&
      width % 8 == 0 && width <= 256 * 8 * 4 && ld_s % 4 == 0 && (!branch || ld_b % 8 == 0) && aligned16(stream_) &&
      (!branch || (aligned16(branch) && aligned16(wb))) && (!out || (aligned16(out) && aligned16(w)))) {
    if (io_dtype == DT_BF16)
      launch_stream_regs<bf16>(branch, ld_b, wb, eps_b, off_b, mult, stream_, ld_s, rows, w, out, eps, off, n_rows, width, stream);
    else
      launch_stream_regs<float>(branch, ld_b, wb, eps_b, off_b, mult, stream_, ld_s, rows, w, out, eps, off, n_rows, width, stream);
    return launch_status();
  }
  if (width > 16384) return ERR_UNSUPPORTED;
  rmsnorm_stream_kernel<<<(unsigned)n_rows, 256, (size_t)width * sizeof(float), stream>>>(
      branch, branch_dtype, ld_b, wb, eps_b, off_b, mult, stream_, stream_dtype, ld_s, rows, w, param_dtype, out,
      out_dtype, eps, off, width);
  return launch_status();
}
