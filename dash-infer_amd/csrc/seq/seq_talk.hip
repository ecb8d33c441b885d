// seq_talk.hip -- grouped-query attention whose softmax maps are mixed between the heads ("talking heads", after the softmax):
//   w_g(i, j) = softmax_j(q_g(i) . k_kv(g)(j) * scale * temp[g])  over the keys j of the row's window,
//   out_h(i)  = sum_j ( sum_g talk[h, g] w_g(i, j) ) v_kv(h)(j)   (* gate[i, h, :])
// The mixed weight of head h needs the NORMALISED weights of every head at the same key, so the softmax cannot run in one
// pass beside the value product.  Two passes over the keys:
//   talk_stats   the maximum and the denominator of every (row, head) -- per part of the key walk, merged by the readers
//   talk_apply   per 64-key chunk: every head's normalised weights -> LDS, the H x H mix per key, the mixed weights times the
//                values of the head's own key/value head.  Weights that are normalised by the final statistics need no
//                rescaling, so the parts of a split key walk simply add up (talk_merge, parts in order).
// Scores, weights, the mix and every sum are f32 for any cache type.  One workgroup per (row, part of the walk): a row's result
// does not depend on what else is in the batch.  Keys and values come from the pages only (the step's own rows were appended
// before).
#include "seq_common.h"

namespace dihip {
namespace {

constexpr int TALK_MAX_H = 64;

struct TalkArgs {
  void* out; int odt; long ldo;
  const float* q; long ldq;
  void* const* kspans; void* const* vspans; int span_stride, span_len;
  const void* temp; const void* talk; int wdt;   // temp [H] (NULL: 1), talk [H, H]
  const float* gate; long ldg;                   // [T, H * DV] multiplier on the output (NULL: none)
  const int32_t* tok_slot; const int32_t* tok_pos;
  int H, G, D, DV; float scale; int window;
  int nsplit; float* stats;                      // [T][nsplit][H][2]
  float* part;                                   // [T][nsplit][H * DV] (nsplit > 1)
};

// the keys [lo, hi) that part s of the walk of the row at position pos reads: whole 64-key chunks counted from the window's start
__device__ __forceinline__ void talk_range(const TalkArgs& a, int pos, int s, int* lo, int* hi) {
  const int w_lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int chunks = (pos - w_lo) / 64 + 1, per = (chunks + a.nsplit - 1) / a.nsplit;
  *lo = min(pos + 1, w_lo + s * per * 64);
  *hi = min(pos + 1, w_lo + (s + 1) * per * 64);
}

template <int CT>
__device__ __forceinline__ float talk_score(const TalkArgs& a, const float* __restrict__ qh, void* const* ktab, int j, int g, float mul) {
  constexpr size_t ES = CT == DIHIP_F32 ? 4 : 2;
  const char* kr = (const char*)ktab[j / a.span_len] + ((size_t)(j % a.span_len) * a.G + g) * a.D * ES;
  float d = 0.f;
  if ((a.D & 7) == 0) {
    for (int r = 0; r < a.D; r += 8) {
      float kv[8];
      if (CT == DIHIP_F32) {
        const f32x4_t k0 = *reinterpret_cast<const f32x4_t*>(kr + (size_t)r * 4), k1 = *reinterpret_cast<const f32x4_t*>(kr + (size_t)r * 4 + 16);
#pragma unroll
        for (int x = 0; x < 4; ++x) { kv[x] = k0[x]; kv[4 + x] = k1[x]; }
      } else {
        const uint4 kk = *reinterpret_cast<const uint4*>(kr + (size_t)r * 2);
        const uint32_t u[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
        for (int x = 0; x < 4; ++x) { kv[2 * x] = __uint_as_float(u[x] << 16); kv[2 * x + 1] = __uint_as_float(u[x] & 0xffff0000u); }
      }
#pragma unroll
      for (int x = 0; x < 8; ++x) d = __builtin_fmaf(qh[r + x], kv[x], d);
    }
  } else {
    for (int r = 0; r < a.D; ++r) d = __builtin_fmaf(qh[r], load_ft<CT>(kr, r), d);
  }
  return d * a.scale * mul;
}

template <int CT>
__global__ __launch_bounds__(256) void talk_stats_kernel(TalkArgs a) {
  const int t = blockIdx.x, s = blockIdx.y, lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pos = a.tok_pos[t], hpg = a.H / a.G;
  int lo, hi;
  talk_range(a, pos, s, &lo, &hi);
  void* const* ktab = a.kspans + (size_t)a.tok_slot[t] * a.span_stride;
  for (int h = wave; h < a.H; h += 4) {
    const float* qh = a.q + (size_t)t * a.ldq + (size_t)h * a.D;
    const float mul = a.temp ? ld_any(a.temp, h, a.wdt) : 1.f;
    float mx = -INFINITY, den = 0.f;
    for (int j0 = lo; j0 < hi; j0 += 64) {
      const int j = j0 + lane;
      const float sc = j < hi ? talk_score<CT>(a, qh, ktab, j, h / hpg, mul) : -INFINITY;
      const float mnew = fmaxf(mx, wave_max(sc));
      const float p = j < hi ? expf(sc - mnew) : 0.f;
      den = (mx == -INFINITY ? 0.f : den * expf(mx - mnew)) + wave_sum(p);
      mx = mnew;
    }
    if (lane == 0) {
      float* st = a.stats + (((size_t)t * a.nsplit + s) * a.H + h) * 2;
      st[0] = mx;
      st[1] = den;
    }
  }
}

// HPW: heads per wave (H <= 4 * HPW), RV: value columns per lane (DV <= 64 * RV)
template <int CT, int HPW, int RV>
__global__ __launch_bounds__(256) void talk_apply_kernel(TalkArgs a) {
  __shared__ float talk_s[TALK_MAX_H * TALK_MAX_H];
  __shared__ float ps[TALK_MAX_H][64];
  __shared__ float pw[4][64];
  __shared__ float mx_s[TALK_MAX_H], inv_s[TALK_MAX_H];
  const int t = blockIdx.x, s = blockIdx.y, lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int H = a.H, DV = a.DV, hpg = H / a.G;
  const int pos = a.tok_pos[t];
  int lo, hi;
  talk_range(a, pos, s, &lo, &hi);
  for (int h = threadIdx.x; h < H; h += 256) {       // the row's statistics over all parts of the walk, parts in order
    const float* st = a.stats + ((size_t)t * a.nsplit * H + h) * 2;
    float mx = -INFINITY;
    for (int x = 0; x < a.nsplit; ++x) mx = fmaxf(mx, st[(size_t)x * H * 2]);
    float den = 0.f;
    for (int x = 0; x < a.nsplit; ++x) {
      const float m = st[(size_t)x * H * 2];
      if (m != -INFINITY) den += st[(size_t)x * H * 2 + 1] * expf(m - mx);
    }
    mx_s[h] = mx;
    inv_s[h] = 1.f / den;
  }
  for (int e = threadIdx.x; e < H * H; e += 256) talk_s[e] = ld_any(a.talk, e, a.wdt);
  void* const* ktab = a.kspans + (size_t)a.tok_slot[t] * a.span_stride;
  void* const* vtab = a.vspans + (size_t)a.tok_slot[t] * a.span_stride;
  constexpr size_t ES = CT == DIHIP_F32 ? 4 : 2;
  float acc[HPW][RV];
#pragma unroll
  for (int i = 0; i < HPW; ++i)
#pragma unroll
    for (int v = 0; v < RV; ++v) acc[i][v] = 0.f;
  __syncthreads();
  for (int j0 = lo; j0 < hi; j0 += 64) {
    const int j = j0 + lane, cnt = min(64, hi - j0);
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      const int h = i * 4 + wave;
      if (h < H) {
        float p = 0.f;
        if (j < hi) {
          const float mul = a.temp ? ld_any(a.temp, h, a.wdt) : 1.f;
          p = expf(talk_score<CT>(a, a.q + (size_t)t * a.ldq + (size_t)h * a.D, ktab, j, h / hpg, mul) - mx_s[h]) * inv_s[h];
        }
        ps[h][lane] = p;
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      const int h = i * 4 + wave;
      float pm = 0.f;
      if (h < H)
        for (int g = 0; g < H; ++g) pm = __builtin_fmaf(talk_s[h * H + g], ps[g][lane], pm);
      pw[wave][lane] = pm;
      __syncthreads();
      if (h < H) {
        const int gv = h / hpg;
        for (int jj = 0; jj < cnt; ++jj) {
          const int jk = j0 + jj;
          const char* vr = (const char*)vtab[jk / a.span_len] + ((size_t)(jk % a.span_len) * a.G + gv) * DV * ES;
          const float pj = pw[wave][jj];
#pragma unroll
          for (int v = 0; v < RV; ++v) {
            const int r = v * 64 + lane;
            if (r < DV) acc[i][v] = __builtin_fmaf(pj, load_ft<CT>(vr, r), acc[i][v]);
          }
        }
      }
      __syncthreads();
    }
  }
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    const int h = i * 4 + wave;
    if (h >= H) continue;
#pragma unroll
    for (int v = 0; v < RV; ++v) {
      const int r = v * 64 + lane;
      if (r >= DV) continue;
      const size_t c = (size_t)h * DV + r;
      if (a.nsplit > 1) a.part[((size_t)t * a.nsplit + s) * H * DV + c] = acc[i][v];
      else st_any(a.out, (size_t)t * a.ldo + c, a.odt, a.gate ? acc[i][v] * a.gate[(size_t)t * a.ldg + c] : acc[i][v]);
    }
  }
}

__global__ __launch_bounds__(256) void talk_merge_kernel(TalkArgs a) {
  const int t = blockIdx.x, N = a.H * a.DV;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < N; c += 256 * gridDim.y) {
    float v = 0.f;
    for (int s = 0; s < a.nsplit; ++s) v += a.part[((size_t)t * a.nsplit + s) * N + c];
    st_any(a.out, (size_t)t * a.ldo + c, a.odt, a.gate ? v * a.gate[(size_t)t * a.ldg + c] : v);
  }
}

}  // namespace
}  // namespace dihip

using namespace dihip;

extern "C" {

size_t dihip_talk_attn_workspace_bytes(int T, int H, int DV, int nsplit) {
  size_t b = (size_t)T * nsplit * H * 2 * sizeof(float);
  if (nsplit > 1) b += (size_t)T * nsplit * H * DV * sizeof(float);
  return b;
}

int dihip_talk_attn(void* stream, void* out, int out_dtype, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                    int span_stride, int span_len, int cache_dtype, const void* temp, const void* talk, int w_dtype, const float* gate, long ldg,
                    const int32_t* tok_slot, const int32_t* tok_pos, int T, int H, int G, int D, int DV, float scale, int window, int nsplit,
                    void* ws, size_t ws_bytes) {
  DIHIP_REQUIRE(T >= 0 && out && q && kspans && vspans && talk && tok_slot && tok_pos && span_stride > 0 && span_len > 0 && H > 0 && G > 0 &&
                    H % G == 0 && D > 0 && DV > 0 && ldo >= (long)H * DV && ldq >= (long)H * D && (!gate || ldg >= (long)H * DV) && nsplit >= 1 &&
                    nsplit <= 65535 && seq_dtype_ok(out_dtype) && seq_dtype_ok(cache_dtype) && seq_dtype_ok(w_dtype),
                DIHIP_PARAM_ERROR, "talk_attn: bad argument");
  DIHIP_REQUIRE(H <= TALK_MAX_H && DV <= 256, DIHIP_EXCEED_LIMIT_ERROR, "talk_attn: at most %d heads and values of at most 256 elements", TALK_MAX_H);
  DIHIP_REQUIRE(ws && ws_bytes >= dihip_talk_attn_workspace_bytes(T, H, DV, nsplit) && (reinterpret_cast<uintptr_t>(ws) & 3u) == 0,
                DIHIP_PARAM_ERROR, "talk_attn: workspace too small");
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  float* stats = (float*)ws;
  TalkArgs a{out, out_dtype, ldo, q, ldq, kspans, vspans, span_stride, span_len, temp, talk, w_dtype, gate, ldg, tok_slot, tok_pos,
             H, G, D, DV, scale, window, nsplit, stats, stats + (size_t)T * nsplit * H * 2};
  const dim3 grid(T, nsplit);
  auto go = [&](auto ct, auto hpw, auto rv) {
    constexpr int CT = decltype(ct)::value, HPW = decltype(hpw)::value, RV = decltype(rv)::value;
    hipLaunchKernelGGL((talk_apply_kernel<CT, HPW, RV>), grid, dim3(256), 0, s, a);
  };
  auto by_rv = [&](auto ct, auto hpw) {
    if (DV <= 64) go(ct, hpw, std::integral_constant<int, 1>{});
    else if (DV <= 128) go(ct, hpw, std::integral_constant<int, 2>{});
    else go(ct, hpw, std::integral_constant<int, 4>{});
  };
  auto by_h = [&](auto ct) {
    if (H <= 4) by_rv(ct, std::integral_constant<int, 1>{});
    else if (H <= 8) by_rv(ct, std::integral_constant<int, 2>{});
    else if (H <= 16) by_rv(ct, std::integral_constant<int, 4>{});
    else if (H <= 32) by_rv(ct, std::integral_constant<int, 8>{});
    else by_rv(ct, std::integral_constant<int, 16>{});
  };
  if (cache_dtype == DIHIP_F32) {
    hipLaunchKernelGGL(talk_stats_kernel<DIHIP_F32>, grid, dim3(256), 0, s, a);
    by_h(std::integral_constant<int, DIHIP_F32>{});
  } else {
    hipLaunchKernelGGL(talk_stats_kernel<DIHIP_BF16>, grid, dim3(256), 0, s, a);
    by_h(std::integral_constant<int, DIHIP_BF16>{});
  }
  if (nsplit > 1) hipLaunchKernelGGL(talk_merge_kernel, dim3(T, T >= 256 ? 1 : (H * DV + 1023) / 1024), dim3(256), 0, s, a);
  return launch_status();
}

}  // extern "C"
