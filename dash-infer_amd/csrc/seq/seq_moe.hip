// seq_moe.hip -- routing and glue of the mixture-of-experts feed-forward (the expert products are dihip_linear_segmented):
//   moe_route      per token, f32: the `top` experts of largest router logit (ties: the lower index), weights = softmax over the
//                  chosen logits alone; or (scoring 1) scores = softmax over ALL logits, the choice by score + a correction per
//                  expert, weights = the chosen scores over their sum
//   moe_sort       the (token, choice) pairs grouped by expert in a fixed order: segment bounds per expert, the token each
//                  sorted row reads, and where each pair went
//   moe_glu        the experts' activation on [gate | up] rows (clamped sigmoid unit, or silu(gate) * up)
//   moe_combine    out[t] = sum over the token's choices, in order, of weight * the expert's output row -- the token's own input
//                  row for the experts past the real ones (identity experts) -- plus an optional row added for every token
#include "seq_common.h"

namespace dihip {
namespace {

// One token's choice.  scoring 0: the `top` largest logits (ties: the lower index), weights = softmax over them alone.  scoring 1:
// scores = softmax over all E logits, the choice by score + correction, weights = the chosen scores over their sum.  (Every logit
// is read a few times: E is small and the row stays in cache.)
template <int SCORING>
__device__ __forceinline__ void route_token(const float* __restrict__ z, const void* __restrict__ corr, int cdt, int E, int top, int ngroups,
                                            int keep, int (&bi)[32], float (&w)[32]) {
  float zmax = -INFINITY, den = 1.f;
  if (SCORING == 1) {
    for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, z[e]);
    den = 0.f;
    for (int e = 0; e < E; ++e) den += expf(z[e] - zmax);
  }
  // group-limited choice: the experts form ngroups equal groups of neighbours, a group counts by its best expert, and only the
  // experts of the `keep` best groups (ties: the lower index) can be chosen
  uint32_t open_groups = 0xffffffffu;
  const int gsz = ngroups > 1 ? E / ngroups : E;
  if (ngroups > 1 && keep < ngroups) {
    open_groups = 0u;
    for (int k = 0; k < keep; ++k) {
      float bv = -INFINITY;
      int bg = -1;
      for (int g = 0; g < ngroups; ++g) {
        if (open_groups >> g & 1u) continue;
        float gv = -INFINITY;
        for (int e = g * gsz; e < (g + 1) * gsz; ++e) gv = fmaxf(gv, SCORING == 1 ? expf(z[e] - zmax) / den : z[e]);
        if (bg < 0 || gv > bv) { bv = gv; bg = g; }
      }
      open_groups |= 1u << bg;
    }
  }
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY, bs = 0.f;
    int bx = -1;
    for (int e = 0; e < E; ++e) {
      bool used = false;
      for (int j = 0; j < k; ++j) used |= bi[j] == e;
      float v = z[e], sc = v;
      if (SCORING == 1) {
        sc = expf(v - zmax) / den;
        v = sc + (corr ? ld_any(corr, e, cdt) : 0.f);
      }
      if (ngroups > 1 && !(open_groups >> (e / gsz) & 1u)) used = true;
      if (!used && (bx < 0 || v > bv)) { bv = v; bx = e; bs = sc; }
    }
    w[k] = bs; bi[k] = bx;
    sum += bs;
  }
  if (SCORING == 1) {
    for (int k = 0; k < top; ++k) w[k] = w[k] / (sum + 1e-20f);
  } else {
    float d = 0.f;
    const float m0 = w[0];
    for (int k = 0; k < top; ++k) { w[k] = expf(w[k] - m0); d += w[k]; }
    for (int k = 0; k < top; ++k) w[k] = w[k] / d;
  }
}

template <int SCORING>
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, long ldl, const void* __restrict__ corr, int cdt,
                                                        int32_t* __restrict__ ids, float* __restrict__ wts, int T, int E, int top, int ngroups, int keep) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= T) return;
  int bi[32];
  float w[32];
  route_token<SCORING>(logits + (size_t)t * ldl, corr, cdt, E, top, ngroups, keep, bi, w);
  for (int k = 0; k < top; ++k) {
    ids[(size_t)t * top + k] = bi[k];
    wts[(size_t)t * top + k] = w[k];
  }
}

// Few pairs (T * top <= 1024, E <= 256; decoding): the choice, the counts and the places in ONE workgroup -- the same ids, weights
// and row order as the three launches below.
template <int SCORING>
__global__ __launch_bounds__(256) void moe_route_small_kernel(const float* __restrict__ logits, long ldl, const void* __restrict__ corr, int cdt,
                                                              int32_t* __restrict__ ids, float* __restrict__ wts, int32_t* __restrict__ counts,
                                                              int32_t* __restrict__ seg, int32_t* __restrict__ src_row, int32_t* __restrict__ dst,
                                                              int T, int E, int top, int ngroups, int keep) {
  __shared__ int ids_s[1024];
  __shared__ int cnt_s[256];
  const int tid = threadIdx.x, R = T * top;
  for (int t = tid; t < T; t += 256) {
    int bi[32];
    float w[32];
    route_token<SCORING>(logits + (size_t)t * ldl, corr, cdt, E, top, ngroups, keep, bi, w);
    for (int k = 0; k < top; ++k) {
      ids[(size_t)t * top + k] = ids_s[t * top + k] = bi[k];
      wts[(size_t)t * top + k] = w[k];
    }
  }
  __syncthreads();
  int c = 0;
  if (tid < E) {
    for (int r = 0; r < R; ++r) c += ids_s[r] == tid;
    cnt_s[tid] = c;
    counts[tid] = c;
  }
  __syncthreads();
  if (tid < E) {
    int pos = 0;
    for (int x = 0; x < tid; ++x) pos += cnt_s[x];
    seg[tid] = pos;
    if (tid == E - 1) seg[E] = pos + c;
    for (int r = 0; r < R; ++r)
      if (ids_s[r] == tid) {
        src_row[pos] = r / top;
        dst[r] = pos;
        ++pos;
      }
  }
}

// block e: how many pairs chose expert e
__global__ __launch_bounds__(256) void moe_count_kernel(const int32_t* __restrict__ ids, int R, int32_t* __restrict__ counts) {
  __shared__ int red[4];
  const int e = blockIdx.x;
  int c = 0;
  for (int r = threadIdx.x; r < R; r += 256) c += ids[r] == e;
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) counts[e] = red[0] + red[1] + red[2] + red[3];
}

// block e: its pairs in ascending pair order -> sorted rows seg[e] ..; thread i scans the pairs [i * per, (i + 1) * per)
__global__ __launch_bounds__(256) void moe_place_kernel(const int32_t* __restrict__ ids, int R, int top, int E, const int32_t* __restrict__ counts,
                                                        int32_t* __restrict__ seg, int32_t* __restrict__ src_row, int32_t* __restrict__ dst) {
  __shared__ int scan[256];
  const int e = blockIdx.x, tid = threadIdx.x;
  const int per = (R + 255) / 256, lo = min(R, tid * per), hi = min(R, lo + per);
  int c = 0;
  for (int r = lo; r < hi; ++r) c += ids[r] == e;
  scan[tid] = c;
  __syncthreads();
  int base = 0;
  for (int x = 0; x < e; ++x) base += counts[x];
  if (tid == 0) {
    seg[e] = base;
    if (e == E - 1) seg[E] = base + counts[e];
  }
  int before = 0;
  for (int x = 0; x < tid; ++x) before += scan[x];
  int pos = base + before;
  for (int r = lo; r < hi; ++r)
    if (ids[r] == e) {
      src_row[pos] = r / top;
      dst[r] = pos;
      ++pos;
    }
}

__global__ __launch_bounds__(256) void moe_glu_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ gu, long ldgu, int F,
                                                      float limit, float slope, int unit) {
  const int r = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < F; c += 256 * gridDim.y) {
    if (unit == 1) {      // silu(gate) * up
      const float g = gu[(size_t)r * ldgu + c], u = gu[(size_t)r * ldgu + F + c];
      st_any(y, (size_t)r * ldy + c, ydt, g / (1.f + expf(-g)) * u);
      continue;
    }
    const float g = fminf(gu[(size_t)r * ldgu + c], limit);
    const float u = fminf(fmaxf(gu[(size_t)r * ldgu + F + c], -limit), limit);
    st_any(y, (size_t)r * ldy + c, ydt, g * (1.f / (1.f + expf(-slope * g))) * (u + 1.f));
  }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ out, long ldo, const float* __restrict__ rows, long ldr,
                                                          const int32_t* __restrict__ dst, const float* __restrict__ wts, int top, int K,
                                                          const int32_t* __restrict__ ids, int n_real, const void* __restrict__ own, int odt,
                                                          long ldown, const float* __restrict__ add, long ldadd) {
  const int t = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < K; c += 256 * gridDim.y) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const size_t pr = (size_t)t * top + k;
      const float v = ids && ids[pr] >= n_real ? ld_any(own, (size_t)t * ldown + c, odt) : rows[(size_t)dst[pr] * ldr + c];
      acc = __builtin_fmaf(wts[pr], v, acc);
    }
    if (add) acc += add[(size_t)t * ldadd + c];
    out[(size_t)t * ldo + c] = acc;
  }
}

}  // namespace
}  // namespace dihip

using namespace dihip;

extern "C" {

int dihip_seq_moe_route(void* stream, const float* logits, long ldl, int32_t* ids, float* wts, int32_t* counts, int32_t* seg, int32_t* src_row,
                    int32_t* dst, int T, int E, int top, int scoring, const void* correction, int w_dtype, int ngroups, int keep) {
  DIHIP_REQUIRE(ngroups >= 1 && ngroups <= 32 && E % ngroups == 0 && keep >= 1 && keep <= ngroups && (long)keep * (E / ngroups) >= top,
                DIHIP_PARAM_ERROR, "moe_route: at most 32 equal groups, of which the kept ones must hold the choices");
  DIHIP_REQUIRE((scoring == 0 || scoring == 1) && (!correction || scoring == 1) && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR,
                "moe_route: unknown scoring (a correction goes with scoring 1)");
  DIHIP_REQUIRE(T >= 0 && E > 0 && top > 0 && top <= E && top <= 32 && E <= 65535 && logits && ids && wts && counts && seg && src_row && dst &&
                    ldl >= E, DIHIP_PARAM_ERROR, "moe_route: bad argument (at most 32 choices per token)");
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if ((long)T * top <= 1024 && E <= 256) {
    if (scoring == 1) hipLaunchKernelGGL(moe_route_small_kernel<1>, dim3(1), dim3(256), 0, s, logits, ldl, correction, w_dtype, ids, wts, counts, seg, src_row, dst, T, E, top, ngroups, keep);
    else hipLaunchKernelGGL(moe_route_small_kernel<0>, dim3(1), dim3(256), 0, s, logits, ldl, correction, w_dtype, ids, wts, counts, seg, src_row, dst, T, E, top, ngroups, keep);
    return launch_status();
  }
  if (scoring == 1) hipLaunchKernelGGL(moe_route_kernel<1>, dim3((T + 255) / 256), dim3(256), 0, s, logits, ldl, correction, w_dtype, ids, wts, T, E, top, ngroups, keep);
  else hipLaunchKernelGGL(moe_route_kernel<0>, dim3((T + 255) / 256), dim3(256), 0, s, logits, ldl, correction, w_dtype, ids, wts, T, E, top, ngroups, keep);
  hipLaunchKernelGGL(moe_count_kernel, dim3(E), dim3(256), 0, s, ids, T * top, counts);
  hipLaunchKernelGGL(moe_place_kernel, dim3(E), dim3(256), 0, s, ids, T * top, top, E, counts, seg, src_row, dst);
  return launch_status();
}

int dihip_seq_moe_glu(void* stream, void* y, int y_dtype, long ldy, const float* gu, long ldgu, int R, int F, float limit, float slope, int unit) {
  DIHIP_REQUIRE((unit == 0 || unit == 1) && R >= 0 && F > 0 && y && gu && ldy >= F && ldgu >= 2 * (long)F && seq_dtype_ok(y_dtype), DIHIP_PARAM_ERROR, "moe_glu: bad argument");
  if (R == 0) return DIHIP_SUCCESS;
  hipLaunchKernelGGL(moe_glu_kernel, dim3(R, R >= 256 ? 1 : (F + 1023) / 1024), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), y, y_dtype, ldy, gu, ldgu, F, limit, slope, unit);
  return launch_status();
}

int dihip_seq_moe_combine(void* stream, float* out, long ldo, const float* rows, long ldr, const int32_t* dst, const float* wts, int T, int top,
                      int K, const int32_t* ids, int n_real, const void* own, int own_dtype, long ldown, const float* add, long ldadd) {
  DIHIP_REQUIRE(T >= 0 && top > 0 && K > 0 && out && rows && dst && wts && ldo >= K && ldr >= K, DIHIP_PARAM_ERROR, "moe_combine: bad argument");
  DIHIP_REQUIRE((!ids || (own && ldown >= K && seq_dtype_ok(own_dtype) && n_real >= 0)) && (!add || ldadd >= K), DIHIP_PARAM_ERROR,
                "moe_combine: identity experts need the tokens' own rows; added rows at least K wide");
  if (T == 0) return DIHIP_SUCCESS;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T, T >= 256 ? 1 : (K + 1023) / 1024), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), out, ldo, rows, ldr, dst, wts, top, K, ids, n_real, own, own_dtype, ldown, add, ldadd);
  return launch_status();
}

}  // extern "C"
