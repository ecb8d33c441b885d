// seq_mixers.hip -- the token-mixing and residual-stream operators of the sequence engine (everything in f32):
// embedding sums, strided RMS norms (also into the paged latent cache), the output-normed residual step with the
// depth-weighted stream, windowed sink-softmax attention over shared latent rows, causal short convolutions and the
// gated linear recurrence with per-slot state.
#include <cstdarg>
#include <cstdio>

#include "seq_common.h"

namespace dihip {
namespace {

// ------------------------------------------------------------------------------------------------ embedding
template <int WT>
__global__ __launch_bounds__(256) void embed_sum_kernel(float* __restrict__ h, const int32_t* __restrict__ ids, const void* __restrict__ table,
                                                        const int32_t* __restrict__ rows2, const void* __restrict__ table2, int K) {
  const int t = blockIdx.x;
  const size_t r1 = (size_t)ids[t] * K, r2 = table2 ? (size_t)rows2[t] * K : 0;
  const bool two = table2 != nullptr;
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) {
    float v = load_ft<WT>(table, r1 + k);
    if (two) v += load_ft<WT>(table2, r2 + k);
    h[(size_t)t * K + k] = v;
  }
}

// columns [col0, col0 + K) of the table rows ids[t], times a constant, into rows of any stride and type
template <int WT>
__global__ __launch_bounds__(256) void embed_rows_kernel(void* __restrict__ y, int ydt, long ldy, const int32_t* __restrict__ ids,
                                                         const void* __restrict__ table, long ldt, long col0, float scale, int K) {
  const int t = blockIdx.x;
  const size_t r = (size_t)ids[t] * ldt + col0;
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) st_any(y, (size_t)t * ldy + k, ydt, load_ft<WT>(table, r + k) * scale);
}

// ------------------------------------------------------------------------------------------------ norms
// sum of squares of a row, k ascending per thread, one fixed tree over the block
__device__ __forceinline__ float row_sumsq(const float* __restrict__ x, int K, float* red) {
  float ss = 0.f;
  if ((K & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0) {   // (block-uniform) 16-byte loads, four of them in flight
#pragma unroll 4
    for (int k = threadIdx.x * 4; k < K; k += 1024) {
      const f32x4_t v = *reinterpret_cast<const f32x4_t*>(x + k);
      ss = __builtin_fmaf(v[0], v[0], ss);
      ss = __builtin_fmaf(v[1], v[1], ss);
      ss = __builtin_fmaf(v[2], v[2], ss);
      ss = __builtin_fmaf(v[3], v[3], ss);
    }
  } else {
#pragma unroll 8
    for (int k = threadIdx.x; k < K; k += 256) {
      const float v = x[k];
      ss = __builtin_fmaf(v, v, ss);
    }
  }
  return block256_sum(ss, red);
}

template <int WT>
__global__ __launch_bounds__(256) void rmsnorm_strided_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ x, long ldx,
                                                              const int32_t* __restrict__ row_idx, const void* __restrict__ gamma,
                                                              float gamma_add, float out_scale, float eps, int K) {
  __shared__ float red[4];
  const int i = blockIdx.x;
  const float* xr = x + (size_t)(row_idx ? row_idx[i] : i) * ldx;
  const float inv = 1.f / sqrtf(row_sumsq(xr, K, red) / (float)K + eps);
  if (gamma_add == 0.f && out_scale == 1.f) {
#pragma unroll 4
    for (int k = threadIdx.x; k < K; k += 256) st_any(y, (size_t)i * ldy + k, ydt, xr[k] * inv * load_ft<WT>(gamma, k));
  } else {
#pragma unroll 4
    for (int k = threadIdx.x; k < K; k += 256) st_any(y, (size_t)i * ldy + k, ydt, xr[k] * inv * (gamma_add + load_ft<WT>(gamma, k)) * out_scale);
  }
}

// The residual step of a layer with norms before AND after its sublayers, one workgroup per row:
//   xo = x_in + m / rms(m) * (add_m + gamma_m)   (m NULL: xo = x_in);   x_out = xo;   xc = xo (any type / stride);
//   h  = xo / rms(xo) * (add_h + gamma_h)        (the next sublayer's input norm)
// Every thread re-reads only what it wrote itself.
template <int WT>
__global__ __launch_bounds__(256) void residual_norm_step_kernel(float* x_out, const float* x_in, const float* __restrict__ m, long ldm,
                                                                 const void* __restrict__ gamma_m, float add_m, const void* __restrict__ gamma_h,
                                                                 float add_h, float eps, void* __restrict__ xc, int cdt, long ldc,
                                                                 void* __restrict__ h, int hdt, long ldh, int K) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const size_t row = (size_t)t * K;
  const float* mr = m ? m + (size_t)t * ldm : nullptr;
  float inv_m = 0.f;
  if (m) inv_m = 1.f / sqrtf(row_sumsq(mr, K, red) / (float)K + eps);
  float ss = 0.f;
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) {
    float xo = x_in[row + k];
    if (m) {
      xo += mr[k] * inv_m * (add_m + load_ft<WT>(gamma_m, k));
      x_out[row + k] = xo;
    }
    if (xc) st_any(xc, (size_t)t * ldc + k, cdt, xo);
    ss = __builtin_fmaf(xo, xo, ss);
  }
  if (!h) return;
  const float inv = 1.f / sqrtf(block256_sum(ss, red) / (float)K + eps);
  const float* src = m ? x_out : x_in;
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) st_any(h, (size_t)t * ldh + k, hdt, src[row + k] * inv * (add_h + load_ft<WT>(gamma_h, k)));
}

template <int WT>
__global__ __launch_bounds__(256) void norm_span_append_kernel(void* const* __restrict__ spans, int span_stride, int span_len, int cdt,
                                                               const float* __restrict__ x, long ldx, const void* __restrict__ gamma,
                                                               float eps, const int32_t* __restrict__ tok_slot,
                                                               const int32_t* __restrict__ tok_pos, int K) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float* xr = x + (size_t)t * ldx;
  const float inv = 1.f / sqrtf(row_sumsq(xr, K, red) / (float)K + eps);
  const int pos = tok_pos[t];
  void* span = spans[(size_t)tok_slot[t] * span_stride + pos / span_len];
  const size_t base = (size_t)(pos % span_len) * K;
#pragma unroll 4
  for (int k = threadIdx.x; k < K; k += 256) st_any(span, base + k, cdt, xr[k] * inv * load_ft<WT>(gamma, k));
}

// The depth mix reads every earlier level of the stack: its weights are staged in LDS and the levels are read through a
// restrict view (the level written here is never one of them), so that a thread's loads are all in flight together.
template <int WT>
__global__ __launch_bounds__(256) void norm_residual_mix_kernel(float* x_out, const float* x_in, const float* __restrict__ m,
                                                                long ldm, const void* __restrict__ gamma, float eps,
                                                                float* stack_top, const float* __restrict__ stack, size_t stack_stride,
                                                                const void* __restrict__ mix_w, int n_mix, float* __restrict__ x_mix,
                                                                uint16_t* __restrict__ next16, int K) {
  __shared__ float red[4];
  __shared__ float mw[256];
  const int t = blockIdx.x;
  if (threadIdx.x < n_mix) mw[threadIdx.x] = load_ft<WT>(mix_w, threadIdx.x);
  const float* mr = m + (size_t)t * ldm;
  const float inv = 1.f / sqrtf(row_sumsq(mr, K, red) / (float)K + eps);   // (its barriers publish mw)
  const size_t row = (size_t)t * K;
  for (int k0 = threadIdx.x; k0 < K; k0 += 1024) {
    float xo[4], mix[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + i * 256;
      xo[i] = mix[i] = 0.f;
      if (k < K) {
        xo[i] = x_in[row + k] + mr[k] * inv * load_ft<WT>(gamma, k);
#pragma unroll 4
        for (int j = 0; j + 1 < n_mix; ++j) mix[i] = __builtin_fmaf(mw[j], stack[(size_t)j * stack_stride + row + k], mix[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + i * 256;
      if (k < K) {
        x_out[row + k] = xo[i];
        float nx = xo[i];
        if (n_mix > 0) {
          stack_top[row + k] = xo[i];
          nx = __builtin_fmaf(mw[n_mix - 1], xo[i], mix[i]);
          x_mix[row + k] = nx;
        }
        if (next16) next16[row + k] = (uint16_t)f32_to_bf16_bits(nx);
      }
    }
  }
}

// The norm without statistics and the parallel residual step: x_out = x_in + (a + b), h = tanh(alpha * x_out) * w + bias.
// row_idx: h[i] is the norm of row row_idx[i] (x_out is then not written).
template <int WT>
__global__ __launch_bounds__(256) void add_dyt_kernel(float* x_out, const float* x_in, const float* __restrict__ a, long lda,
                                                      const float* __restrict__ b, long ldb, const int32_t* __restrict__ row_idx, float alpha,
                                                      const void* __restrict__ w, const void* __restrict__ bias, float* __restrict__ h,
                                                      uint16_t* __restrict__ h16, int K) {
  const int i = blockIdx.x;
  const size_t r = row_idx ? (size_t)row_idx[i] : (size_t)i;
  const int k_lo = blockIdx.y * 1024, k_hi = min(K, k_lo + 1024);   // a row's columns are spread over gridDim.y workgroups (few rows: decoding)
#pragma unroll 4
  for (int k = k_lo + threadIdx.x; k < k_hi; k += 256) {
    float v = x_in[r * K + k];
    if (a) {
      float s = a[r * lda + k];
      if (b) s += b[r * ldb + k];
      v += s;
    }
    if (x_out) x_out[r * K + k] = v;
    if (w) {
      const float y = tanhf(alpha * v) * load_ft<WT>(w, k) + load_ft<WT>(bias, k);
      if (h) h[(size_t)i * K + k] = y;
      if (h16) h16[(size_t)i * K + k] = (uint16_t)f32_to_bf16_bits(y);
    }
  }
}

// The same step for rows of up to 1024 * VPT elements (a multiple of 4, 16-byte aligned rows): the row stays in registers, every
// operand is read once and all of a thread's loads are in flight together -- two memory round trips and two block sums per row.
template <int WT, int VPT>
__global__ __launch_bounds__(256) void residual_norm_step_reg_kernel(float* x_out, const float* x_in, const float* __restrict__ m, long ldm,
                                                                     const void* __restrict__ gamma_m, float add_m,
                                                                     const void* __restrict__ gamma_h, float add_h, float eps,
                                                                     void* __restrict__ xc, int cdt, long ldc, void* __restrict__ h, int hdt,
                                                                     long ldh, int K) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const size_t row = (size_t)t * K;
  const f32x4_t z4 = {0.f, 0.f, 0.f, 0.f};
  f32x4_t xv[VPT], mv[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int k = (threadIdx.x + 256 * i) * 4;
    xv[i] = k < K ? *reinterpret_cast<const f32x4_t*>(x_in + row + k) : z4;
    mv[i] = m && k < K ? *reinterpret_cast<const f32x4_t*>(m + (size_t)t * ldm + k) : z4;
  }
  if (m) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) ss = __builtin_fmaf(mv[i][j], mv[i][j], ss);
    const float inv_m = 1.f / sqrtf(block256_sum(ss, red) / (float)K + eps);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int k = (threadIdx.x + 256 * i) * 4;
      if (k < K) {
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[i][j] += mv[i][j] * inv_m * (add_m + load_ft<WT>(gamma_m, k + j));
        *reinterpret_cast<f32x4_t*>(x_out + row + k) = xv[i];
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int k = (threadIdx.x + 256 * i) * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) ss = __builtin_fmaf(xv[i][j], xv[i][j], ss);
    if (xc && k < K) {
#pragma unroll
      for (int j = 0; j < 4; ++j) st_any(xc, (size_t)t * ldc + k + j, cdt, xv[i][j]);
    }
  }
  if (!h) return;
  const float inv = 1.f / sqrtf(block256_sum(ss, red) / (float)K + eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int k = (threadIdx.x + 256 * i) * 4;
    if (k < K) {
#pragma unroll
      for (int j = 0; j < 4; ++j) st_any(h, (size_t)t * ldh + k + j, hdt, xv[i][j] * inv * (add_h + load_ft<WT>(gamma_h, k + j)));
    }
  }
}

// ------------------------------------------------------------------------------------------------ latent attention
// One workgroup per row, its 4 waves take the heads in turn.  A wave walks the row's window in chunks of 64 keys: lane j
// scores key j (f32 dot over the R latent elements, r ascending), the chunk joins the running softmax (which starts at
// the sink: maximum = sink, denominator = 1), then the lanes turn to the latent elements (lane l owns r = l, l + 64, ..)
// and add the chunk's weighted rows.  Keys come from the cache only (the step's own rows were appended before).
template <int CT, int RV>
__global__ __launch_bounds__(256) void latent_attn_kernel(float* __restrict__ out, long ldo, const float* __restrict__ q, long ldq,
                                                          void* const* __restrict__ spans, int span_stride, int span_len,
                                                          const void* __restrict__ sink, int wdt, const int32_t* __restrict__ tok_slot,
                                                          const int32_t* __restrict__ tok_pos, int H, int R, int window, float scale) {
  __shared__ float qs[4][RV * 64];
  __shared__ float ps[4][64];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pos = tok_pos[t];
  const int j_lo = window > 0 ? max(0, pos - window + 1) : 0;
  void* const* tab = spans + (size_t)tok_slot[t] * span_stride;
  constexpr size_t ES = CT == DIHIP_F32 ? 4 : 2;
  for (int h0 = 0; h0 < H; h0 += 4) {
    const int h = h0 + wave;
    const bool live = h < H;
    __syncthreads();  // qs / ps of the head before are no longer read
    if (live)
      for (int r = lane; r < R; r += 64) qs[wave][r] = q[(size_t)t * ldq + (size_t)h * R + r];
    __syncthreads();
    float mx = -INFINITY, den = 0.f;
    if (sink) { mx = ld_any(sink, h < H ? h : 0, wdt); den = 1.f; }
    float acc[RV];
#pragma unroll
    for (int v = 0; v < RV; ++v) acc[v] = 0.f;
    for (int j0 = j_lo; j0 <= pos; j0 += 64) {  // the same trip count in every wave of the block
      const int j = j0 + lane;
      const bool valid = live && j <= pos;
      float s = -INFINITY;
      if (valid) {
        const char* row = (const char*)tab[j / span_len] + (size_t)(j % span_len) * R * ES;
        float d = 0.f;
        for (int r = 0; r < R; ++r) d = __builtin_fmaf(qs[wave][r], load_ft<CT>(row, r), d);
        s = d * scale;
      }
      const float mnew = fmaxf(mx, wave_max(s));
      const float corr = mx == -INFINITY ? 0.f : expf(mx - mnew);
      const float p = valid ? expf(s - mnew) : 0.f;
      den = den * corr + wave_sum(p);
#pragma unroll
      for (int v = 0; v < RV; ++v) acc[v] *= corr;
      mx = mnew;
      ps[wave][lane] = p;
      __syncthreads();
      if (live) {
        const int cnt = min(64, pos - j0 + 1);
        for (int jj = 0; jj < cnt; ++jj) {
          const int jk = j0 + jj;
          const char* row = (const char*)tab[jk / span_len] + (size_t)(jk % span_len) * R * ES;
          const float pj = ps[wave][jj];
#pragma unroll
          for (int v = 0; v < RV; ++v) {
            const int r = v * 64 + lane;
            if (r < R) acc[v] = __builtin_fmaf(pj, load_ft<CT>(row, r), acc[v]);
          }
        }
      }
      __syncthreads();
    }
    if (live) {
#pragma unroll
      for (int v = 0; v < RV; ++v) {
        const int r = v * 64 + lane;
        if (r < R) out[(size_t)t * ldo + (size_t)h * R + r] = acc[v] / den;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ short convolution
__global__ __launch_bounds__(256) void causal_conv_state_kernel(float* __restrict__ u, long ldu, const float* __restrict__ x, long ldx,
                                                                const void* __restrict__ w, const void* __restrict__ bias, int wdt,
                                                                const float* __restrict__ tail, const int32_t* __restrict__ tok_slot,
                                                                const int32_t* __restrict__ tok_off, int C, int taps, int silu) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int off = tok_off[t], nt = taps - 1;
  const float* tl = tail + (size_t)tok_slot[t] * nt * C;
  float acc = 0.f;
  for (int k = 0; k < taps; ++k) {
    const int d = nt - k, o = off - d;
    const float v = o >= 0 ? x[(size_t)(t - d) * ldx + c] : tl[(size_t)(nt + o) * C + c];
    acc = __builtin_fmaf(ld_any(w, (size_t)c * taps + k, wdt), v, acc);
  }
  if (bias) acc += ld_any(bias, c, wdt);
  if (silu) acc = acc / (1.f + expf(-acc));
  u[(size_t)t * ldu + c] = acc;
}

__global__ __launch_bounds__(256) void conv_tail_update_kernel(float* __restrict__ tail, const float* __restrict__ x, long ldx,
                                                               const int32_t* __restrict__ ent_slot, const int32_t* __restrict__ ent_row0,
                                                               const int32_t* __restrict__ ent_count, int C, int taps) {
  const int e = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int nt = taps - 1, cnt = ent_count[e], row0 = ent_row0[e];
  float* tl = tail + (size_t)ent_slot[e] * nt * C;
  float old[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) old[i] = i < nt ? tl[(size_t)i * C + c] : 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if (i < nt) {
      const int o = cnt - nt + i;  // index inside the portion of the input that becomes tail row i
      float v;
      if (o >= 0) v = x[(size_t)(row0 + o) * ldx + c];
      else {
        v = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j)
          if (j == nt + o) v = old[j];
      }
      tl[(size_t)i * C + c] = v;
    }
  }
}

// ------------------------------------------------------------------------------------------------ gated recurrence
__device__ __forceinline__ float softplus_f32(float x) { return x > 20.f ? x : log1pf(expf(x)); }

__global__ __launch_bounds__(64) void gated_recurrence_kernel(float* __restrict__ out, long ldo, const float* __restrict__ r, const float* __restrict__ ig,
                                                              long ldg, const float* __restrict__ u, long ldu, const float* __restrict__ y, long ldy,
                                                              const void* __restrict__ lam, int wdt, float decay, float* __restrict__ state,
                                                              const int32_t* __restrict__ ent_slot, const int32_t* __restrict__ ent_row0,
                                                              const int32_t* __restrict__ ent_count, int C) {
  const int e = blockIdx.x, c = blockIdx.y * 64 + threadIdx.x;
  if (c >= C) return;
  const int cnt = ent_count[e], row0 = ent_row0[e];
  float* sp = state + (size_t)ent_slot[e] * C + c;
  float S = *sp;
  const float k = -decay * softplus_f32(ld_any(lam, c, wdt));
  constexpr int U = 8;
  for (int i0 = 0; i0 < cnt; i0 += U) {
    float rv[U], iv[U], uv[U], yv[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const size_t t = (size_t)(row0 + min(i0 + j, cnt - 1));
      rv[j] = r[t * ldg + c]; iv[j] = ig[t * ldg + c]; uv[j] = u[t * ldu + c]; yv[j] = y[t * ldy + c];
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      if (i0 + j < cnt) {
        const float la = k * rv[j];
        const float a = expf(la);
        const float g = sqrtf(-expm1f(2.f * la)) * iv[j] * uv[j];
        S = __builtin_fmaf(a, S, g);
        out[(size_t)(row0 + i0 + j) * ldo + c] = S * yv[j];
      }
    }
  }
  *sp = S;
}

// Long portions: the recurrence S_t = a_t S_(t-1) + g_t is a composition of affine maps, so a portion is cut into chunks of
// REC_CHUNK rows that run side by side.  Pass 1: every (chunk, channel) composes its rows from S = 0: (A = prod a_t, B = the
// state it would end in).  Pass 2 (per channel, chunks in order): the state each chunk really starts from, S <- A S + B.
// Pass 3: every chunk runs its rows from that state and writes the outputs.  The cut changes the result by f32 rounding only.
constexpr int REC_CHUNK = 64;

struct RecArgs {
  float* out; long ldo; const float* r; const float* ig; long ldg; const float* u; long ldu; const float* y; long ldy;
  const void* lam; int wdt; float decay; float* state; const int32_t* ent_slot; const int32_t* ent_row0; const int32_t* ent_count;
  int C; float* ab; int max_chunks;   // ab: [E][max_chunks][2][C]
};

template <int PASS>
__global__ __launch_bounds__(64) void gated_recurrence_chunk_kernel(RecArgs a) {
  const int e = blockIdx.z, ch = blockIdx.x, c = blockIdx.y * 64 + threadIdx.x;
  const int cnt = a.ent_count[e], row0 = a.ent_row0[e];
  const int lo = ch * REC_CHUNK;
  if (c >= a.C || lo >= cnt) return;
  const int n = min(REC_CHUNK, cnt - lo);
  float* ab = a.ab + ((size_t)e * a.max_chunks + ch) * 2 * a.C;
  const float k = -a.decay * softplus_f32(ld_any(a.lam, c, a.wdt));
  float S = PASS == 1 ? 0.f : ab[c], A = 1.f;
  constexpr int U = 8;
  for (int i0 = 0; i0 < n; i0 += U) {
    float rv[U], iv[U], uv[U], yv[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const size_t t = (size_t)(row0 + lo + min(i0 + j, n - 1));
      rv[j] = a.r[t * a.ldg + c]; iv[j] = a.ig[t * a.ldg + c]; uv[j] = a.u[t * a.ldu + c];
      if (PASS == 3) yv[j] = a.y[t * a.ldy + c];
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      if (i0 + j < n) {
        const float la = k * rv[j];
        const float av = expf(la);
        S = __builtin_fmaf(av, S, sqrtf(-expm1f(2.f * la)) * iv[j] * uv[j]);
        if (PASS == 1) A *= av;
        else a.out[(size_t)(row0 + lo + i0 + j) * a.ldo + c] = S * yv[j];
      }
    }
  }
  if (PASS == 1) { ab[c] = A; ab[a.C + c] = S; }
  else if (lo + n == cnt) a.state[(size_t)a.ent_slot[e] * a.C + c] = S;
}

// pass 2: ab[ch][0] <- the state chunk ch starts from
__global__ __launch_bounds__(64) void gated_recurrence_carry_kernel(RecArgs a) {
  const int e = blockIdx.x, c = blockIdx.y * 64 + threadIdx.x;
  if (c >= a.C) return;
  const int chunks = (a.ent_count[e] + REC_CHUNK - 1) / REC_CHUNK;
  float S = a.state[(size_t)a.ent_slot[e] * a.C + c];
  for (int ch = 0; ch < chunks; ++ch) {
    float* ab = a.ab + ((size_t)e * a.max_chunks + ch) * 2 * a.C;
    const float A = ab[c], B = ab[a.C + c];
    ab[c] = S;
    S = __builtin_fmaf(A, S, B);
  }
}

static thread_local char g_seq_error[512] = "";

}  // namespace

void set_last_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_seq_error, sizeof(g_seq_error), fmt, ap);
  va_end(ap);
}
int env_int(const char* name, int dflt) {
  const char* e = getenv(name);
  return e ? atoi(e) : dflt;
}
bool env_off(const char* name) {
  const char* e = getenv(name);
  return e && e[0] == '0';
}

}  // namespace dihip

using namespace dihip;

extern "C" {

const char* dihip_seq_version(void) { return "dashinfer-hip-seq 0.1.0 (gfx950)"; }
const char* dihip_seq_last_error(void) { return g_seq_error; }

int dihip_embed_sum(void* stream, float* h, const int32_t* ids, const void* table, const int32_t* rows2, const void* table2,
                    int w_dtype, int T, int K) {
  DIHIP_REQUIRE(T >= 0 && K > 0 && h && ids && table && (!table2 || rows2) && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "embed_sum: bad argument");
  if (T == 0) return DIHIP_SUCCESS;
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(embed_sum_kernel<DIHIP_F32>, dim3(T), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), h, ids, table, rows2, table2, K);
  else hipLaunchKernelGGL(embed_sum_kernel<DIHIP_BF16>, dim3(T), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), h, ids, table, rows2, table2, K);
  return launch_status();
}

int dihip_embed_rows(void* stream, void* y, int y_dtype, long ldy, const int32_t* ids, const void* table, int w_dtype, long ldt, long col0,
                     float scale, int T, int K) {
  DIHIP_REQUIRE(T >= 0 && K > 0 && y && ids && table && ldy >= K && col0 >= 0 && ldt >= col0 + K && seq_dtype_ok(w_dtype) && seq_dtype_ok(y_dtype),
                DIHIP_PARAM_ERROR, "embed_rows: bad argument");
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(embed_rows_kernel<DIHIP_F32>, dim3(T), dim3(256), 0, s, y, y_dtype, ldy, ids, table, ldt, col0, scale, K);
  else hipLaunchKernelGGL(embed_rows_kernel<DIHIP_BF16>, dim3(T), dim3(256), 0, s, y, y_dtype, ldy, ids, table, ldt, col0, scale, K);
  return launch_status();
}

int dihip_residual_norm_step(void* stream, float* x_out, const float* x_in, const float* m, long ldm, const void* gamma_m, float add_m,
                             const void* gamma_h, float add_h, int w_dtype, float eps, void* xc, int xc_dtype, long ldc, void* h, int h_dtype,
                             long ldh, int T, int K) {
  DIHIP_REQUIRE(T >= 0 && K > 0 && x_in && (!m || (x_out && gamma_m && ldm >= K)) && (!h || (gamma_h && ldh >= K)) && (!xc || ldc >= K) &&
                    seq_dtype_ok(w_dtype) && seq_dtype_ok(xc_dtype) && seq_dtype_ok(h_dtype), DIHIP_PARAM_ERROR, "residual_norm_step: bad argument");
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (K % 4 == 0 && K <= 8192 && al16(x_in) && (!m || (al16(m) && ldm % 4 == 0 && al16(x_out)))) {   // the row fits the registers
    auto go = [&](auto wt, auto vpt) {
      constexpr int WT = decltype(wt)::value, VPT = decltype(vpt)::value;
      hipLaunchKernelGGL((residual_norm_step_reg_kernel<WT, VPT>), dim3(T), dim3(256), 0, s, x_out, x_in, m, ldm, gamma_m, add_m, gamma_h, add_h, eps,
                         xc, xc_dtype, ldc, h, h_dtype, ldh, K);
    };
    auto by_k = [&](auto wt) {
      if (K <= 1024) go(wt, std::integral_constant<int, 1>{});
      else if (K <= 2048) go(wt, std::integral_constant<int, 2>{});
      else if (K <= 4096) go(wt, std::integral_constant<int, 4>{});
      else go(wt, std::integral_constant<int, 8>{});
    };
    if (w_dtype == DIHIP_F32) by_k(std::integral_constant<int, DIHIP_F32>{});
    else by_k(std::integral_constant<int, DIHIP_BF16>{});
    return launch_status();
  }
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(residual_norm_step_kernel<DIHIP_F32>, dim3(T), dim3(256), 0, s, x_out, x_in, m, ldm, gamma_m, add_m, gamma_h, add_h, eps, xc, xc_dtype, ldc, h, h_dtype, ldh, K);
  else hipLaunchKernelGGL(residual_norm_step_kernel<DIHIP_BF16>, dim3(T), dim3(256), 0, s, x_out, x_in, m, ldm, gamma_m, add_m, gamma_h, add_h, eps, xc, xc_dtype, ldc, h, h_dtype, ldh, K);
  return launch_status();
}

int dihip_rmsnorm_strided(void* stream, void* y, int y_dtype, long ldy, const float* x, long ldx, const int32_t* row_idx,
                          const void* gamma, int w_dtype, float gamma_add, float out_scale, float eps, int M, int K) {
  DIHIP_REQUIRE(M >= 0 && K > 0 && y && x && gamma && ldy >= K && ldx >= K && seq_dtype_ok(y_dtype) && seq_dtype_ok(w_dtype),
                DIHIP_PARAM_ERROR, "rmsnorm_strided: bad argument");
  if (M == 0) return DIHIP_SUCCESS;
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(rmsnorm_strided_kernel<DIHIP_F32>, dim3(M), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), y, y_dtype, ldy, x, ldx, row_idx, gamma, gamma_add, out_scale, eps, K);
  else hipLaunchKernelGGL(rmsnorm_strided_kernel<DIHIP_BF16>, dim3(M), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), y, y_dtype, ldy, x, ldx, row_idx, gamma, gamma_add, out_scale, eps, K);
  return launch_status();
}

int dihip_norm_span_append(void* stream, void* const* spans, int span_stride, int span_len, int cache_dtype, const float* x, long ldx,
                           const void* gamma, int w_dtype, float eps, const int32_t* tok_slot, const int32_t* tok_pos, int T, int K) {
  DIHIP_REQUIRE(T >= 0 && K > 0 && spans && x && gamma && tok_slot && tok_pos && span_stride > 0 && span_len > 0 && ldx >= K &&
                    seq_dtype_ok(cache_dtype) && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "norm_span_append: bad argument");
  if (T == 0) return DIHIP_SUCCESS;
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(norm_span_append_kernel<DIHIP_F32>, dim3(T), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), spans, span_stride, span_len, cache_dtype, x, ldx, gamma, eps, tok_slot, tok_pos, K);
  else hipLaunchKernelGGL(norm_span_append_kernel<DIHIP_BF16>, dim3(T), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), spans, span_stride, span_len, cache_dtype, x, ldx, gamma, eps, tok_slot, tok_pos, K);
  return launch_status();
}

int dihip_norm_residual_mix(void* stream, float* x_out, const float* x_in, const float* m, long ldm, const void* gamma, int w_dtype,
                            float eps, float* stack, size_t stack_stride, const void* mix_w, int n_mix, float* x_mix, void* next16, int T,
                            int K) {
  DIHIP_REQUIRE(T >= 0 && K > 0 && x_out && x_in && m && gamma && ldm >= K && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR,
                "norm_residual_mix: bad argument");
  DIHIP_REQUIRE(n_mix == 0 || (stack && mix_w && x_mix && stack_stride >= (size_t)T * K && x_mix != x_out), DIHIP_PARAM_ERROR,
                "norm_residual_mix: the depth mix needs the stack, its weights and an output of its own");
  if (T == 0) return DIHIP_SUCCESS;
  DIHIP_REQUIRE(n_mix <= 256, DIHIP_EXCEED_LIMIT_ERROR, "norm_residual_mix: more than 256 levels");
  float* top = n_mix > 0 ? stack + (size_t)(n_mix - 1) * stack_stride : nullptr;
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(norm_residual_mix_kernel<DIHIP_F32>, dim3(T), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), x_out, x_in, m, ldm, gamma, eps, top, stack, stack_stride, mix_w, n_mix, x_mix, (uint16_t*)next16, K);
  else hipLaunchKernelGGL(norm_residual_mix_kernel<DIHIP_BF16>, dim3(T), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), x_out, x_in, m, ldm, gamma, eps, top, stack, stack_stride, mix_w, n_mix, x_mix, (uint16_t*)next16, K);
  return launch_status();
}

int dihip_add_dyt(void* stream, float* x_out, const float* x_in, const float* a, long lda, const float* b, long ldb, const int32_t* row_idx,
                  float alpha, const void* w, const void* bias, int w_dtype, float* h, void* h16, int M, int K) {
  DIHIP_REQUIRE(M >= 0 && K > 0 && x_in && (!a || lda >= K) && (!b || (a && ldb >= K)) && (!w || bias) && (!row_idx || !x_out) &&
                    seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "add_dyt: bad argument");
  if (M == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(add_dyt_kernel<DIHIP_F32>, dim3(M, (K + 1023) / 1024), dim3(256), 0, s, x_out, x_in, a, lda, b, ldb, row_idx, alpha, w, bias, h, (uint16_t*)h16, K);
  else hipLaunchKernelGGL(add_dyt_kernel<DIHIP_BF16>, dim3(M, (K + 1023) / 1024), dim3(256), 0, s, x_out, x_in, a, lda, b, ldb, row_idx, alpha, w, bias, h, (uint16_t*)h16, K);
  return launch_status();
}

int dihip_latent_window_attn(void* stream, float* out, long ldo, const float* q, long ldq, void* const* spans, int span_stride,
                             int span_len, int cache_dtype, const void* sink, int w_dtype, const int32_t* tok_slot,
                             const int32_t* tok_pos, int T, int H, int R, int window, float scale, int math) {
  DIHIP_REQUIRE(T >= 0 && H > 0 && R > 0 && out && q && spans && tok_slot && tok_pos && span_stride > 0 && span_len > 0 &&
                    ldo >= (long)H * R && ldq >= (long)H * R && seq_dtype_ok(cache_dtype) && seq_dtype_ok(w_dtype),
                DIHIP_PARAM_ERROR, "latent_window_attn: bad argument");
  DIHIP_REQUIRE(R <= 1024, DIHIP_EXCEED_LIMIT_ERROR, "latent_window_attn: latent rows of more than 1024 elements (%d)", R);
  (void)math;
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  auto go = [&](auto ct, auto rv) {
    constexpr int CT = decltype(ct)::value, RV = decltype(rv)::value;
    hipLaunchKernelGGL((latent_attn_kernel<CT, RV>), dim3(T), dim3(256), 0, s, out, ldo, q, ldq, spans, span_stride, span_len, sink,
                       w_dtype, tok_slot, tok_pos, H, R, window, scale);
  };
  auto by_r = [&](auto ct) {
    if (R <= 64) go(ct, std::integral_constant<int, 1>{});
    else if (R <= 128) go(ct, std::integral_constant<int, 2>{});
    else if (R <= 256) go(ct, std::integral_constant<int, 4>{});
    else if (R <= 512) go(ct, std::integral_constant<int, 8>{});
    else go(ct, std::integral_constant<int, 16>{});
  };
  if (cache_dtype == DIHIP_F32) by_r(std::integral_constant<int, DIHIP_F32>{});
  else by_r(std::integral_constant<int, DIHIP_BF16>{});
  return launch_status();
}

int dihip_causal_conv_state(void* stream, float* u, long ldu, const float* x, long ldx, const void* w, const void* bias, int w_dtype,
                            const float* tail, const int32_t* tok_slot, const int32_t* tok_off, int T, int C, int taps, int act) {
  DIHIP_REQUIRE(T >= 0 && C > 0 && taps >= 1 && taps <= 16 && u && x && w && (tail || taps == 1) && tok_slot && tok_off && ldu >= C &&
                    ldx >= C && seq_dtype_ok(w_dtype) && (act == 0 || act == 5), DIHIP_PARAM_ERROR,
                "causal_conv_state: bad argument (1 <= taps <= 16; activation none or silu)");
  if (T == 0) return DIHIP_SUCCESS;
  hipLaunchKernelGGL(causal_conv_state_kernel, dim3(T, (C + 255) / 256), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), u, ldu, x, ldx,
                     w, bias, w_dtype, tail, tok_slot, tok_off, C, taps, act == 5);
  return launch_status();
}

int dihip_conv_tail_update(void* stream, float* tail, const float* x, long ldx, const int32_t* ent_slot, const int32_t* ent_row0,
                           const int32_t* ent_count, int E, int C, int taps) {
  DIHIP_REQUIRE(E >= 0 && C > 0 && taps >= 1 && taps <= 16 && x && ent_slot && ent_row0 && ent_count && ldx >= C, DIHIP_PARAM_ERROR,
                "conv_tail_update: bad argument (1 <= taps <= 16)");
  if (E == 0 || taps == 1) return DIHIP_SUCCESS;
  DIHIP_REQUIRE(tail, DIHIP_PARAM_ERROR, "conv_tail_update: null state");
  hipLaunchKernelGGL(conv_tail_update_kernel, dim3(E, (C + 255) / 256), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), tail, x, ldx,
                     ent_slot, ent_row0, ent_count, C, taps);
  return launch_status();
}

size_t dihip_gated_recurrence_chunked_workspace_bytes(int E, int max_count, int C) {
  return (size_t)E * ((max_count + REC_CHUNK - 1) / REC_CHUNK) * 2 * C * sizeof(float);
}

int dihip_gated_recurrence_chunked(void* stream, float* out, long ldo, const float* r, const float* i, long ldg, const float* u, long ldu,
                                   const float* y, long ldy, const void* lam, int w_dtype, float decay, float* state,
                                   const int32_t* ent_slot, const int32_t* ent_row0, const int32_t* ent_count, int E, int max_count, int C,
                                   void* ws, size_t ws_bytes) {
  DIHIP_REQUIRE(E >= 0 && max_count >= 0 && C > 0 && out && r && i && u && y && lam && state && ent_slot && ent_row0 && ent_count &&
                    ldo >= C && ldg >= C && ldu >= C && ldy >= C && seq_dtype_ok(w_dtype) && E <= 65535, DIHIP_PARAM_ERROR,
                "gated_recurrence_chunked: bad argument");
  DIHIP_REQUIRE(ws && ws_bytes >= dihip_gated_recurrence_chunked_workspace_bytes(E, max_count, C), DIHIP_PARAM_ERROR,
                "gated_recurrence_chunked: workspace too small");
  if (E == 0 || max_count == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int chunks = (max_count + REC_CHUNK - 1) / REC_CHUNK;
  RecArgs a{out, ldo, r, i, ldg, u, ldu, y, ldy, lam, w_dtype, decay, state, ent_slot, ent_row0, ent_count, C, (float*)ws, chunks};
  const dim3 grid(chunks, (C + 63) / 64, E);
  hipLaunchKernelGGL(gated_recurrence_chunk_kernel<1>, grid, dim3(64), 0, s, a);
  hipLaunchKernelGGL(gated_recurrence_carry_kernel, dim3(E, (C + 63) / 64), dim3(64), 0, s, a);
  hipLaunchKernelGGL(gated_recurrence_chunk_kernel<3>, grid, dim3(64), 0, s, a);
  return launch_status();
}

int dihip_gated_recurrence(void* stream, float* out, long ldo, const float* r, const float* i, long ldg, const float* u, long ldu,
                           const float* y, long ldy, const void* lam, int w_dtype, float decay, float* state, const int32_t* ent_slot,
                           const int32_t* ent_row0, const int32_t* ent_count, int E, int C) {
  DIHIP_REQUIRE(E >= 0 && C > 0 && out && r && i && u && y && lam && state && ent_slot && ent_row0 && ent_count && ldo >= C &&
                    ldg >= C && ldu >= C && ldy >= C && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "gated_recurrence: bad argument");
  if (E == 0) return DIHIP_SUCCESS;
  hipLaunchKernelGGL(gated_recurrence_kernel, dim3(E, (C + 63) / 64), dim3(64), 0, reinterpret_cast<hipStream_t>(stream), out, ldo, r, i, ldg,
                     u, ldu, y, ldy, lam, w_dtype, decay, state, ent_slot, ent_row0, ent_count, C);
  return launch_status();
}

}  // extern "C"
