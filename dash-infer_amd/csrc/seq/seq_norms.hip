// seq_norms.hip -- row operators of layers that run their sublayers side by side on a layer-normed stream (everything in f32):
//   residual_layernorm   x_out = x_in + mult * (a + b);  h = (x_out - mean) / sqrt(var + eps) * w (+ bias)  -- the residual step of
//                        two sublayers and the NEXT layer's input norm in one launch; with row_idx: the norm of chosen rows alone
//   polynorm             y = c0 z / rms(z) + c1 z^2 / rms(z^2) + c2 z^3 / rms(z^3) + c3   (powers per element, rms over the row)
//   rmsnorm_pair         y = coef * (xa / rms(xa) * wa + xb / rms(xb) * wb)   -- two branches joined on equal footing
//   gate_group_rmsnorm   v = (o + skip[head] * x) * silu(z);  y = v / rms_group(v) * w   -- the gate comes before the norm, the norm
//                        runs over `groups` equal parts of the row
//   latent_rope_append   attention through a latent with one rotated key part shared by the heads: the latent is RMS-normed and
//                        written to its page with the rotated key part behind it (zero padded to the cache row); the rotated
//                        part of every head's query is written behind the head's absorbed query
// One workgroup per row, one fixed reduction tree: a row's result does not depend on the batch it is computed in.
#include "seq_common.h"

namespace dihip {
namespace {

template <int WT>
__global__ __launch_bounds__(256) void residual_layernorm_kernel(float* x_out, const float* x_in, const float* __restrict__ a, long lda,
                                                                 const float* __restrict__ b, long ldb, float mult,
                                                                 const int32_t* __restrict__ row_idx, const void* __restrict__ w,
                                                                 const void* __restrict__ bias, float eps, void* __restrict__ h, int hdt,
                                                                 long ldh, int K) {
  __shared__ float red[4];
  const int i = blockIdx.x;
  const size_t r = row_idx ? (size_t)row_idx[i] : (size_t)i;
  const float* src = x_in + r * K;
  float sum = 0.f;
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) {
    float v = x_in[r * K + k];
    if (a) {
      float s = a[r * lda + k];
      if (b) s += b[r * ldb + k];
      v = __builtin_fmaf(mult, s, v);
    }
    if (x_out) x_out[r * K + k] = v;     // (re-read below by the thread that wrote it)
    sum += v;
  }
  if (!w) return;
  if (x_out) src = x_out + r * K;
  const float mean = block256_sum(sum, red) / (float)K;
  float ss = 0.f;
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) {
    const float d = src[k] - mean;
    ss = __builtin_fmaf(d, d, ss);
  }
  const float inv = 1.f / sqrtf(block256_sum(ss, red) / (float)K + eps);
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) {
    float y = (src[k] - mean) * inv * load_ft<WT>(w, k);
    if (bias) y += load_ft<WT>(bias, k);
    st_any(h, (size_t)i * ldh + k, hdt, y);
  }
}

template <int WT>
__global__ __launch_bounds__(256) void polynorm_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ z, long ldz,
                                                       const void* __restrict__ coef, float eps, int F) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float* zr = z + (size_t)t * ldz;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll 4
  for (int k = threadIdx.x; k < F; k += 256) {
    const float v = zr[k], v2 = v * v, v3 = v2 * v;
    s1 = __builtin_fmaf(v, v, s1);
    s2 = __builtin_fmaf(v2, v2, s2);
    s3 = __builtin_fmaf(v3, v3, s3);
  }
  const float c0 = load_ft<WT>(coef, 0) / sqrtf(block256_sum(s1, red) / (float)F + eps);
  const float c1 = load_ft<WT>(coef, 1) / sqrtf(block256_sum(s2, red) / (float)F + eps);
  const float c2 = load_ft<WT>(coef, 2) / sqrtf(block256_sum(s3, red) / (float)F + eps);
  const float c3 = load_ft<WT>(coef, 3);
#pragma unroll 4
  for (int k = threadIdx.x; k < F; k += 256) {
    const float v = zr[k], v2 = v * v;
    st_any(y, (size_t)t * ldy + k, ydt, c0 * v + c1 * v2 + c2 * (v2 * v) + c3);
  }
}

template <int WT>
__global__ __launch_bounds__(256) void rmsnorm_pair_kernel(float* __restrict__ y, long ldy, const float* __restrict__ xa, long lda,
                                                           const void* __restrict__ wa, const float* __restrict__ xb, long ldb,
                                                           const void* __restrict__ wb, float coef, float eps, int K) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float* ar = xa + (size_t)t * lda;
  const float* br = xb + (size_t)t * ldb;
  float sa = 0.f, sb = 0.f;
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) {
    sa = __builtin_fmaf(ar[k], ar[k], sa);
    sb = __builtin_fmaf(br[k], br[k], sb);
  }
  const float ia = 1.f / sqrtf(block256_sum(sa, red) / (float)K + eps);
  const float ib = 1.f / sqrtf(block256_sum(sb, red) / (float)K + eps);
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256)
    y[(size_t)t * ldy + k] = coef * (ar[k] * ia * load_ft<WT>(wa, k) + br[k] * ib * load_ft<WT>(wb, k));
}

// grid (rows, groups): a workgroup owns one part of one row
template <int WT>
__global__ __launch_bounds__(256) void gate_group_rmsnorm_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ o, long ldo,
                                                                 const float* __restrict__ x, long ldx, const void* __restrict__ skip,
                                                                 const float* __restrict__ z, long ldz, const void* __restrict__ w,
                                                                 float eps, int P, int part) {
  __shared__ float red[4];
  const int t = blockIdx.x, c0 = blockIdx.y * part;
  float ss = 0.f;
#pragma unroll 4
  for (int k = threadIdx.x; k < part; k += 256) {
    const int c = c0 + k;
    float v = o[(size_t)t * ldo + c];
    if (skip) v = __builtin_fmaf(load_ft<WT>(skip, c / P), x[(size_t)t * ldx + c], v);
    const float g = z[(size_t)t * ldz + c];
    v *= g / (1.f + expf(-g));
    ss = __builtin_fmaf(v, v, ss);
  }
  const float inv = 1.f / sqrtf(block256_sum(ss, red) / (float)part + eps);
#pragma unroll 4
  for (int k = threadIdx.x; k < part; k += 256) {     // the same expressions as above: the same bits
    const int c = c0 + k;
    float v = o[(size_t)t * ldo + c];
    if (skip) v = __builtin_fmaf(load_ft<WT>(skip, c / P), x[(size_t)t * ldx + c], v);
    const float g = z[(size_t)t * ldz + c];
    v *= g / (1.f + expf(-g));
    st_any(y, (size_t)t * ldy + c, ydt, v * inv * load_ft<WT>(w, c));
  }
}

// ------------------------------------------------------------------------------------------------ register forms
// A row (or a part of one) of at most NT * EPT elements is loaded ONCE, every load issued before the first use (indices past the
// end are clamped, so no load hangs on a condition), and stays in registers through the reductions.  Rows of more than 1024
// elements take 512 or 1024 threads: with few rows in the step a row's time is the length of one thread's chain of dependent
// instructions, and a looping thread of 256 walks 16 elements of a 4096-wide row one after the other, twice or three times.  The
// form is chosen by the row's length alone, so a row's bits do not depend on the batch.
template <int NW>
__device__ __forceinline__ float tree_sum(const float* r) {
  if constexpr (NW == 1) return r[0];
  else return tree_sum<NW / 2>(r) + tree_sum<NW / 2>(r + NW / 2);
}
// sum over the NT threads of a block, the same value in every thread; red = NT / 64 floats of LDS; one fixed tree
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();  // red may still be read from the call before
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return tree_sum<NT / 64>(red);
}

template <int WT, int NT, int EPT>
__global__ __launch_bounds__(NT) void residual_layernorm_reg_kernel(float* x_out, const float* x_in, const float* __restrict__ a, long lda,
                                                                    const float* __restrict__ b, long ldb, float mult,
                                                                    const int32_t* __restrict__ row_idx, const void* __restrict__ w,
                                                                    const void* __restrict__ bias, float eps, void* __restrict__ h, int hdt,
                                                                    long ldh, int K) {
  __shared__ float red[NT / 64];
  const int i = blockIdx.x, tid = threadIdx.x;
  const size_t r = row_idx ? (size_t)row_idx[i] : (size_t)i;
  float v[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) v[e] = x_in[r * K + min(tid + e * NT, K - 1)];
  if (a) {
    float s[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) s[e] = a[r * lda + min(tid + e * NT, K - 1)];
    if (b) {
#pragma unroll
      for (int e = 0; e < EPT; ++e) s[e] += b[r * ldb + min(tid + e * NT, K - 1)];
    }
#pragma unroll
    for (int e = 0; e < EPT; ++e) v[e] = __builtin_fmaf(mult, s[e], v[e]);
  }
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int k = tid + e * NT;
    if (k < K) {
      if (x_out) x_out[r * K + k] = v[e];
      sum += v[e];
    }
  }
  if (!w) return;
  float g[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) g[e] = load_ft<WT>(w, min(tid + e * NT, K - 1));
  const float mean = block_sum<NT>(sum, red) / (float)K;
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const float d = v[e] - mean;
    if (tid + e * NT < K) ss = __builtin_fmaf(d, d, ss);
  }
  const float inv = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)K + eps);
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int k = tid + e * NT;
    if (k < K) {
      float y = (v[e] - mean) * inv * g[e];
      if (bias) y += load_ft<WT>(bias, k);
      st_any(h, (size_t)i * ldh + k, hdt, y);
    }
  }
}

template <int WT, int NT, int EPT>
__global__ __launch_bounds__(NT) void polynorm_reg_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ z, long ldz,
                                                          const void* __restrict__ coef, float eps, int F) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* zr = z + (size_t)t * ldz;
  float v[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) v[e] = zr[min(tid + e * NT, F - 1)];
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e)
    if (tid + e * NT < F) {
      const float v2 = v[e] * v[e], v3 = v2 * v[e];
      s1 = __builtin_fmaf(v[e], v[e], s1);
      s2 = __builtin_fmaf(v2, v2, s2);
      s3 = __builtin_fmaf(v3, v3, s3);
    }
  const float c0 = load_ft<WT>(coef, 0) / sqrtf(block_sum<NT>(s1, red) / (float)F + eps);
  const float c1 = load_ft<WT>(coef, 1) / sqrtf(block_sum<NT>(s2, red) / (float)F + eps);
  const float c2 = load_ft<WT>(coef, 2) / sqrtf(block_sum<NT>(s3, red) / (float)F + eps);
  const float c3 = load_ft<WT>(coef, 3);
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int k = tid + e * NT;
    if (k < F) {
      const float v2 = v[e] * v[e];
      st_any(y, (size_t)t * ldy + k, ydt, c0 * v[e] + c1 * v2 + c2 * (v2 * v[e]) + c3);
    }
  }
}

template <int WT, int NT, int EPT>
__global__ __launch_bounds__(NT) void rmsnorm_pair_reg_kernel(float* __restrict__ y, long ldy, const float* __restrict__ xa, long lda,
                                                              const void* __restrict__ wa, const float* __restrict__ xb, long ldb,
                                                              const void* __restrict__ wb, float coef, float eps, int K) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, tid = threadIdx.x;
  float va[EPT], vb[EPT], ga[EPT], gb[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int k = min(tid + e * NT, K - 1);
    va[e] = xa[(size_t)t * lda + k];
    vb[e] = xb[(size_t)t * ldb + k];
    ga[e] = load_ft<WT>(wa, k);
    gb[e] = load_ft<WT>(wb, k);
  }
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e)
    if (tid + e * NT < K) {
      sa = __builtin_fmaf(va[e], va[e], sa);
      sb = __builtin_fmaf(vb[e], vb[e], sb);
    }
  const float ia = 1.f / sqrtf(block_sum<NT>(sa, red) / (float)K + eps);
  const float ib = 1.f / sqrtf(block_sum<NT>(sb, red) / (float)K + eps);
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int k = tid + e * NT;
    if (k < K) y[(size_t)t * ldy + k] = coef * (va[e] * ia * ga[e] + vb[e] * ib * gb[e]);
  }
}

// grid (rows, groups): a workgroup owns one part of one row
template <int WT, int NT, int EPT>
__global__ __launch_bounds__(NT) void gate_group_rmsnorm_reg_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ o, long ldo,
                                                                    const float* __restrict__ x, long ldx, const void* __restrict__ skip,
                                                                    const float* __restrict__ z, long ldz, const void* __restrict__ w,
                                                                    float eps, int P, int part) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, c0 = blockIdx.y * part, tid = threadIdx.x;
  float v[EPT], g[EPT], wv[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int c = c0 + min(tid + e * NT, part - 1);
    v[e] = o[(size_t)t * ldo + c];
    g[e] = z[(size_t)t * ldz + c];
    wv[e] = load_ft<WT>(w, c);
  }
  if (skip) {
    float xs[EPT], sk[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int c = c0 + min(tid + e * NT, part - 1);
      xs[e] = x[(size_t)t * ldx + c];
      sk[e] = load_ft<WT>(skip, c / P);
    }
#pragma unroll
    for (int e = 0; e < EPT; ++e) v[e] = __builtin_fmaf(sk[e], xs[e], v[e]);
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    v[e] *= g[e] / (1.f + expf(-g[e]));
    if (tid + e * NT < part) ss = __builtin_fmaf(v[e], v[e], ss);
  }
  const float inv = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)part + eps);
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int k = tid + e * NT;
    if (k < part) st_any(y, (size_t)t * ldy + c0 + k, ydt, v[e] * inv * wv[e]);
  }
}

// ckv: rows [R latent | rot shared key part]; q_rot: rows [H][rot]; ql: rows [H][Rp], the absorbed queries in the first R columns
// of every head.  Rotation of the two halves of the rot dimensions: (u, v) -> (u cos - v sin, v cos + u sin), angle = pos * freq[i].
template <int WT>
__global__ __launch_bounds__(256) void latent_rope_append_kernel(void* const* __restrict__ spans, int span_stride, int span_len, int cdt,
                                                                 const float* __restrict__ ckv, long ldc, const void* __restrict__ gamma,
                                                                 float eps, int R, int rot, int Rp, const float* __restrict__ freq,
                                                                 const float* __restrict__ q_rot, long ldqr, float* __restrict__ ql, long ldql,
                                                                 int H, const int32_t* __restrict__ tok_slot,
                                                                 const int32_t* __restrict__ tok_pos) {
  __shared__ float red[4];
  __shared__ float cs[256], sn[256];
  const int t = blockIdx.x, half = rot >> 1;
  const int pos = tok_pos[t];
  for (int i = threadIdx.x; i < half; i += 256) {
    rope_sincos((uint32_t)pos, freq[i], &sn[i], &cs[i]);
  }
  __syncthreads();
  if (spans) {
    const float* cr = ckv + (size_t)t * ldc;
    float ss = 0.f;
    for (int k = threadIdx.x; k < R; k += 256) ss = __builtin_fmaf(cr[k], cr[k], ss);
    const float inv = 1.f / sqrtf(block256_sum(ss, red) / (float)R + eps);
    void* span = spans[(size_t)tok_slot[t] * span_stride + pos / span_len];
    const size_t base = (size_t)(pos % span_len) * Rp;
    for (int k = threadIdx.x; k < Rp; k += 256) {
      float v = 0.f;
      if (k < R) v = cr[k] * inv * load_ft<WT>(gamma, k);
      else if (k < R + rot) {
        const int i = k - R, j = i < half ? i : i - half;
        const float u = cr[R + j], w = cr[R + half + j];
        v = i < half ? u * cs[j] - w * sn[j] : w * cs[j] + u * sn[j];
      }
      st_any(span, base + k, cdt, v);
    }
  }
  for (int e = threadIdx.x; e < H * rot; e += 256) {
    const int h = e / rot, i = e - h * rot, j = i < half ? i : i - half;
    const float u = q_rot[(size_t)t * ldqr + (size_t)h * rot + j], w = q_rot[(size_t)t * ldqr + (size_t)h * rot + half + j];
    ql[(size_t)t * ldql + (size_t)h * Rp + R + i] = i < half ? u * cs[j] - w * sn[j] : w * cs[j] + u * sn[j];
  }
}

}  // namespace
}  // namespace dihip

using namespace dihip;

#define BY_WT(kernel, wdt, ...)                                              \
  do {                                                                       \
    if ((wdt) == DIHIP_F32) hipLaunchKernelGGL(kernel<DIHIP_F32>, __VA_ARGS__); \
    else hipLaunchKernelGGL(kernel<DIHIP_BF16>, __VA_ARGS__);                \
  } while (0)

// the register form of `kernel` that holds n elements per workgroup, or the looping form (256 threads) beyond 16384
#define BY_WT_ROW(kernel, n, wdt, grid, stream, ...)                                                                     \
  do {                                                                                                                   \
    if ((n) <= 1024) BY_WT_REG(kernel##_reg_kernel, 256, 4, wdt, grid, stream, __VA_ARGS__);                             \
    else if ((n) <= 2048) BY_WT_REG(kernel##_reg_kernel, 512, 4, wdt, grid, stream, __VA_ARGS__);                        \
    else if ((n) <= 4096) BY_WT_REG(kernel##_reg_kernel, 1024, 4, wdt, grid, stream, __VA_ARGS__);                       \
    else if ((n) <= 8192) BY_WT_REG(kernel##_reg_kernel, 1024, 8, wdt, grid, stream, __VA_ARGS__);                       \
    else if ((n) <= 16384) BY_WT_REG(kernel##_reg_kernel, 1024, 16, wdt, grid, stream, __VA_ARGS__);                     \
    else BY_WT(kernel##_kernel, wdt, grid, dim3(256), 0, stream, __VA_ARGS__);                                           \
  } while (0)
#define BY_WT_REG(kernel, NT, EPT, wdt, grid, stream, ...)                                                               \
  do {                                                                                                                   \
    if ((wdt) == DIHIP_F32) hipLaunchKernelGGL((kernel<DIHIP_F32, NT, EPT>), grid, dim3(NT), 0, stream, __VA_ARGS__);    \
    else hipLaunchKernelGGL((kernel<DIHIP_BF16, NT, EPT>), grid, dim3(NT), 0, stream, __VA_ARGS__);                      \
  } while (0)

extern "C" {

int dihip_residual_layernorm(void* stream, float* x_out, const float* x_in, const float* a, long lda, const float* b, long ldb, float mult,
                             const int32_t* row_idx, const void* w, const void* bias, int w_dtype, float eps, void* h, int h_dtype, long ldh,
                             int M, int K) {
  DIHIP_REQUIRE(M >= 0 && K > 0 && x_in && (!a || lda >= K) && (!b || (a && ldb >= K)) && (!w || (h && ldh >= K)) && (!row_idx || !x_out) &&
                    (x_out || !a) && seq_dtype_ok(w_dtype) && seq_dtype_ok(h_dtype), DIHIP_PARAM_ERROR, "residual_layernorm: bad argument");
  if (M == 0) return DIHIP_SUCCESS;
  BY_WT_ROW(residual_layernorm, K, w_dtype, dim3(M), reinterpret_cast<hipStream_t>(stream), x_out, x_in, a, lda, b, ldb, mult, row_idx, w, bias,
            eps, h, h_dtype, ldh, K);
  return launch_status();
}

int dihip_polynorm(void* stream, void* y, int y_dtype, long ldy, const float* z, long ldz, const void* coef, int w_dtype, float eps, int T,
                   int F) {
  DIHIP_REQUIRE(T >= 0 && F > 0 && y && z && coef && ldy >= F && ldz >= F && seq_dtype_ok(y_dtype) && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR,
                "polynorm: bad argument");
  if (T == 0) return DIHIP_SUCCESS;
  BY_WT_ROW(polynorm, F, w_dtype, dim3(T), reinterpret_cast<hipStream_t>(stream), y, y_dtype, ldy, z, ldz, coef, eps, F);
  return launch_status();
}

int dihip_rmsnorm_pair(void* stream, float* y, long ldy, const float* xa, long lda, const void* wa, const float* xb, long ldb, const void* wb,
                       int w_dtype, float coef, float eps, int T, int K) {
  DIHIP_REQUIRE(T >= 0 && K > 0 && y && xa && wa && xb && wb && ldy >= K && lda >= K && ldb >= K && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR,
                "rmsnorm_pair: bad argument");
  if (T == 0) return DIHIP_SUCCESS;
  BY_WT_ROW(rmsnorm_pair, K, w_dtype, dim3(T), reinterpret_cast<hipStream_t>(stream), y, ldy, xa, lda, wa, xb, ldb, wb, coef, eps, K);
  return launch_status();
}

int dihip_gate_group_rmsnorm(void* stream, void* y, int y_dtype, long ldy, const float* o, long ldo, const float* x, long ldx, const void* skip,
                             const float* z, long ldz, const void* w, int w_dtype, float eps, int T, int heads, int P, int groups) {
  const long inner = (long)heads * P;
  DIHIP_REQUIRE(T >= 0 && heads > 0 && P > 0 && groups > 0 && inner % groups == 0 && groups <= 65535 && y && o && z && w && (!skip || x) &&
                    ldy >= inner && ldo >= inner && ldz >= inner && (!skip || ldx >= inner) && seq_dtype_ok(y_dtype) && seq_dtype_ok(w_dtype),
                DIHIP_PARAM_ERROR, "gate_group_rmsnorm: bad argument (the row must divide into the groups)");
  if (T == 0) return DIHIP_SUCCESS;
  BY_WT_ROW(gate_group_rmsnorm, inner / groups, w_dtype, dim3(T, groups), reinterpret_cast<hipStream_t>(stream), y, y_dtype, ldy, o, ldo, x, ldx,
            skip, z, ldz, w, eps, P, (int)(inner / groups));
  return launch_status();
}

int dihip_latent_rope_append(void* stream, void* const* spans, int span_stride, int span_len, int cache_dtype, const float* ckv, long ldc,
                             const void* gamma, int w_dtype, float eps, int R, int rot, int Rp, const float* freq, const float* q_rot, long ldqr,
                             float* ql, long ldql, int H, const int32_t* tok_slot, const int32_t* tok_pos, int T) {
  DIHIP_REQUIRE(T >= 0 && R > 0 && rot >= 0 && rot % 2 == 0 && rot <= 512 && Rp >= R + rot && H > 0 && q_rot && ql && tok_slot && tok_pos &&
                    (rot == 0 || freq) && ldqr >= (long)H * rot && ldql >= (long)H * Rp && seq_dtype_ok(cache_dtype) && seq_dtype_ok(w_dtype),
                DIHIP_PARAM_ERROR, "latent_rope_append: bad argument (an even number of at most 512 rotated dimensions)");
  DIHIP_REQUIRE(!spans || (ckv && gamma && ldc >= R + rot && span_stride > 0 && span_len > 0), DIHIP_PARAM_ERROR,
                "latent_rope_append: a cache needs the rows to append and the norm's weight");
  if (T == 0) return DIHIP_SUCCESS;
  BY_WT(latent_rope_append_kernel, w_dtype, dim3(T), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), spans, span_stride, span_len, cache_dtype,
        ckv, ldc, gamma, eps, R, rot, Rp, freq, q_rot, ldqr, ql, ldql, H, tok_slot, tok_pos);
  return launch_status();
}

}  // extern "C"
