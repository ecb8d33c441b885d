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
#pragma unroll 4
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
  __shared__ const char* vrow_s[64];
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
    if (threadIdx.x < 64) {                            // the chunk's value rows (key/value head 0), published by the barrier below
      const int jk = j0 + threadIdx.x;
      vrow_s[threadIdx.x] = jk < hi ? (const char*)vtab[jk / a.span_len] + (size_t)(jk % a.span_len) * a.G * DV * ES : nullptr;
    }
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
        const size_t voff = (size_t)(h / hpg) * DV * ES;
        for (int jj = 0; jj < cnt; jj += 8) {        // eight keys' loads in flight; the sums run in key order
          float pj[8], vv[8][RV];
#pragma unroll
          for (int x = 0; x < 8; ++x) {
            const bool in = jj + x < cnt;
            const char* vr = in ? vrow_s[jj + x] + voff : nullptr;
            pj[x] = in ? pw[wave][jj + x] : 0.f;
#pragma unroll
            for (int v = 0; v < RV; ++v) {
              const int r = v * 64 + lane;
              vv[x][v] = in && r < DV ? load_ft<CT>(vr, r) : 0.f;
            }
          }
#pragma unroll
          for (int x = 0; x < 8; ++x)
            if (jj + x < cnt) {
#pragma unroll
              for (int v = 0; v < RV; ++v) acc[i][v] = __builtin_fmaf(pj[x], vv[x][v], acc[i][v]);
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

// ------------------------------------------------------------------------------------------------ few rows (decoding)
// With few rows one workgroup per (row, part of the walk) leaves the chip empty and every wave waits on one load after the other.
// The same two passes spread over the heads:
//   talk_scores   one wave per (row, head, 64-key chunk of the row's window): the raw scores -> S [row][head][key], the chunk's
//                 maximum and denominator -> stats
//   talk_mix      one workgroup per (row, OUTPUT head, 256 keys): all heads' statistics merged (chunks in order), the mixed weight of
//                 every key from S, then the values of the head's key/value head -- 64 keys per wave, eight loads in flight, the four
//                 waves' sums added in order
// and talk_merge adds the parts.
struct TalkFewArgs {
  TalkArgs a;
  float* S; int Wp, nchunk;      // S [T][H][Wp] (Wp = nchunk * 64), stats [T][nchunk][H][2]
};

template <int CT>
__global__ __launch_bounds__(64) void talk_scores_kernel(TalkFewArgs f) {
  const TalkArgs& a = f.a;
  const int t = blockIdx.x, h = blockIdx.y, c = blockIdx.z, lane = threadIdx.x;
  const int pos = a.tok_pos[t];
  const int w_lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int j = w_lo + c * 64 + lane;
  const bool valid = j <= pos;
  void* const* ktab = a.kspans + (size_t)a.tok_slot[t] * a.span_stride;
  float sc = -INFINITY;
  if (valid) sc = talk_score<CT>(a, a.q + (size_t)t * a.ldq + (size_t)h * a.D, ktab, j, h / (a.H / a.G), a.temp ? ld_any(a.temp, h, a.wdt) : 1.f);
  f.S[((size_t)t * a.H + h) * f.Wp + c * 64 + lane] = sc;
  const float mx = wave_max(sc);
  const float sum = wave_sum(valid ? expf(sc - mx) : 0.f);
  if (lane == 0) {
    float* st = a.stats + (((size_t)t * f.nchunk + c) * a.H + h) * 2;
    st[0] = mx;
    st[1] = sum;
  }
}

template <int CT, int RV>
__global__ __launch_bounds__(256) void talk_mix_kernel(TalkFewArgs f) {
  const TalkArgs& a = f.a;
  __shared__ float mx_s[TALK_MAX_H], inv_s[TALK_MAX_H], talk_s[TALK_MAX_H];
  __shared__ float pm_s[256];
  __shared__ const char* vrow_s[256];
  __shared__ float red_s[4][64 * RV];
  const int t = blockIdx.x, h = blockIdx.y, part = blockIdx.z, tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int H = a.H, DV = a.DV;
  const int pos = a.tok_pos[t];
  const int w_lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int nch = (pos - w_lo) / 64 + 1;                       // chunks of this row
  for (int g = tid; g < H; g += 256) {       // every load unconditional: the loads of a round are in flight together
    talk_s[g] = ld_any(a.talk, (size_t)h * H + g, a.wdt);
    const float* st = a.stats + ((size_t)t * f.nchunk * H + g) * 2;
    float mx = -INFINITY;
#pragma unroll 8
    for (int c = 0; c < nch; ++c) mx = fmaxf(mx, st[(size_t)c * H * 2]);
    float den = 0.f;
#pragma unroll 8
    for (int c = 0; c < nch; ++c) {
      const float m = st[(size_t)c * H * 2], sm = st[(size_t)c * H * 2 + 1];
      den += m != -INFINITY ? sm * expf(m - mx) : 0.f;
    }
    mx_s[g] = mx;
    inv_s[g] = 1.f / den;
  }
  __syncthreads();
  constexpr size_t ES = CT == DIHIP_F32 ? 4 : 2;
  const int k = part * 256 + tid, j = w_lo + k;                // this thread's key, counted from the window's start
  const bool valid = j <= pos;
  float pm = 0.f;
  if (valid) {
    const float* srow = f.S + (size_t)t * H * f.Wp + k;
#pragma unroll 8
    for (int g = 0; g < H; ++g) pm = __builtin_fmaf(talk_s[g], expf(srow[(size_t)g * f.Wp] - mx_s[g]) * inv_s[g], pm);
  }
  pm_s[tid] = pm;
  void* const* vtab = a.vspans + (size_t)a.tok_slot[t] * a.span_stride;
  vrow_s[tid] = valid ? (const char*)vtab[j / a.span_len] + ((size_t)(j % a.span_len) * a.G + h / (H / a.G)) * DV * ES : nullptr;
  __syncthreads();
  float acc[RV];
#pragma unroll
  for (int v = 0; v < RV; ++v) acc[v] = 0.f;
  const int cnt = min(64, pos - (w_lo + part * 256 + wave * 64) + 1);      // live keys of this wave's 64 (<= 0: none)
  for (int jj = 0; jj < cnt; jj += 16) {       // sixteen keys' loads in flight; the sums run in key order
    float pj[16], vv[16][RV];
#pragma unroll
    for (int x = 0; x < 16; ++x) {             // no load hangs on a condition: past the wave's last live key its row is read again
      const int kk = wave * 64 + min(jj + x, cnt - 1);      // with weight 0, and lanes past the value's width read its last column
      const char* vr = vrow_s[kk];
      pj[x] = jj + x < cnt ? pm_s[kk] : 0.f;
#pragma unroll
      for (int v = 0; v < RV; ++v) vv[x][v] = load_ft<CT>(vr, min(v * 64 + lane, DV - 1));
    }
#pragma unroll
    for (int x = 0; x < 16; ++x) {
#pragma unroll
      for (int v = 0; v < RV; ++v) acc[v] = __builtin_fmaf(pj[x], vv[x][v], acc[v]);
    }
  }
#pragma unroll
  for (int v = 0; v < RV; ++v) red_s[wave][v * 64 + lane] = acc[v];
  __syncthreads();
  for (int r = tid; r < DV; r += 256) {
    const float v = ((red_s[0][r] + red_s[1][r]) + red_s[2][r]) + red_s[3][r];
    const size_t c = (size_t)h * DV + r;
    if (a.nsplit > 1) a.part[((size_t)t * a.nsplit + part) * H * DV + c] = v;
    else st_any(a.out, (size_t)t * a.ldo + c, a.odt, a.gate ? v * a.gate[(size_t)t * a.ldg + c] : v);
  }
}


// ------------------------------------------------------------------------------------------------ matrix-core kernel (bf16 pages)
// A workgroup of 8 waves owns 16 consecutive rows of ONE portion and EVERY head, and walks the 16-key tiles those rows can see, the
// tile's keys (pass 2: and values) of all key/value heads staged in LDS.  Per tile every wave scores HPW heads on the matrix cores
// (S^T = K . Q^T, the query fragments held in registers); lane (row, kb) then holds the keys kb * 4 .. + 3 of its row.
//   PASS 1: the running maximum and denominator of every (row, head) -> stats.
//   PASS 2: the normalised weights of all heads go to LDS ([head][row][key] f32); after a barrier a wave mixes, for each of its OPW
//           output heads, the weights of all heads at its lane's four keys (f32, the mixing row through scalar loads), packs them
//           to bf16 and adds O^T += V^T . P^T on the matrix cores (V^T through the transposing LDS read).
// Scoring every head is cheap beside the mix, so with many heads gridDim.z workgroups share a row tile: each scores all heads and
// owns a part of the OUTPUT heads (fewer accumulators per wave).
typedef short bf16x4s_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4_t mfma_bf16t(const u32x4_t& a, const u32x4_t& b, const f32x4_t& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t mfma_bf16k16(const u32x2_t& a, const u32x2_t& b, const f32x4_t& c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(bf16x4s_t, a), __builtin_bit_cast(bf16x4s_t, b), c, 0, 0, 0);
}
typedef const __attribute__((address_space(4))) float* talk_uniform_ptr;   // read-only for the launch, wave-uniform address: scalar loads

struct TalkMcArgs {
  void* out; int odt; long ldo;
  const float* q; long ldq;
  void* const* kspans; void* const* vspans; int span_stride, span_len;
  const void* temp; int wdt; const float* talk32;   // temp [H] (NULL: 1); talk32: f32 [H][H]
  const float* gate; long ldg;
  const int32_t* tok_pos; const int32_t* ent_slot; const int32_t* ent_row0; const int32_t* ent_count;
  int H, G, D, DV; float scale; int window;
  float* stats;                                     // [T][H][2]
};

template <int PASS, int HPW, int OPW, int DMAX, int VMAX>
__global__ __launch_bounds__(512) void talk_attn_mc_kernel(TalkMcArgs a) {
  constexpr int KS = DMAX / 32, DT = VMAX / 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int G = a.G, H = a.H, D = a.D, DV = a.DV, hpg = H / G;
  const int e = blockIdx.y, cnt = a.ent_count[e], row0 = a.ent_row0[e];
  const int r0 = blockIdx.x * 16;
  if (r0 >= cnt) return;
  const int tid = threadIdx.x, lane = tid & 63, ni = lane & 15, kb = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pitchk = (D + 8) * 2, pitchv = (DV + 8) * 2;
  unsigned char* ksm = smem;                                   // [G][16][pitchk]
  unsigned char* vsm = ksm + G * 16 * pitchk;                  // [G][16][pitchv]   (PASS 2)
  float* psm = reinterpret_cast<float*>(vsm + (PASS == 2 ? G * 16 * pitchv : 0));   // [H][16 rows][16 keys]   (PASS 2)
  const int pos0 = a.tok_pos[row0];
  const bool row_ok = r0 + ni < cnt;
  const int tq = min(r0 + ni, cnt - 1), p = pos0 + tq;
  const int p_lo = pos0 + r0, p_hi = pos0 + min(r0 + 15, cnt - 1);
  const int t_lo = (a.window > 0 ? max(0, p_lo - a.window + 1) : 0) >> 4, t_hi = p_hi >> 4;
  void* const* gkp = a.kspans + (size_t)a.ent_slot[e] * a.span_stride;
  void* const* gvp = a.vspans + (size_t)a.ent_slot[e] * a.span_stride;

  // this wave's heads for the scores: wave + 8 i
  u32x4_t qf[HPW][KS];
  float mul[HPW], mrun[HPW], lrun[HPW];
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    const int h = wave + 8 * i;
    mul[i] = a.scale * (a.temp && h < H ? ld_any(a.temp, h, a.wdt) : 1.f);
    mrun[i] = -1e30f;
    lrun[i] = PASS == 1 ? 0.f : 1.f;
    const float* qrow = a.q + (size_t)(row0 + tq) * a.ldq + (size_t)(h < H ? h : 0) * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[i][ks] = u32x4_t{0u, 0u, 0u, 0u};
      const int d0 = ks * 32 + kb * 8;
      if (d0 < D && h < H) {
        const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(qrow + d0);
        const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(qrow + d0 + 4);
        qf[i][ks] = u32x4_t{pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3])};
      }
    }
    if (PASS == 2 && h < H) {
      const float* st = a.stats + ((size_t)(row0 + tq) * H + h) * 2;
      mrun[i] = st[0];
      lrun[i] = 1.f / st[1];
    }
  }
  const f32x4_t z4 = {0.f, 0.f, 0.f, 0.f};
  f32x4_t oacc[OPW][DT];
#pragma unroll
  for (int i = 0; i < OPW; ++i)
#pragma unroll
    for (int t = 0; t < DT; ++t) oacc[i][t] = z4;

  const int uk = D >> 3, uv = DV >> 3;                         // 16-byte units per key row
  for (int tile = t_lo; tile <= t_hi; ++tile) {
    const int key0 = tile * 16, sp = key0 / a.span_len, in = key0 - sp * a.span_len;
    const int live = min(16, p_hi - key0 + 1);                 // keys of the tile that exist (later ones were never written)
    const char* kbp = (const char*)gkp[sp] + (size_t)in * G * D * 2;
    for (int u = tid; u < 16 * G * uk; u += 512) {             // page rows are [key][G][D]
      const int kin = u / (G * uk), rest = u - kin * (G * uk), g = rest / uk, c8 = rest - g * uk;
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (kin < live) v = gload<u32x4_t>(kbp + ((size_t)(kin * G + g) * D + c8 * 8) * 2);
      *reinterpret_cast<u32x4_t*>(ksm + (g * 16 + kin) * pitchk + c8 * 16) = v;
    }
    if (PASS == 2) {
      const char* vbp = (const char*)gvp[sp] + (size_t)in * G * DV * 2;
      for (int u = tid; u < 16 * G * uv; u += 512) {
        const int kin = u / (G * uv), rest = u - kin * (G * uv), g = rest / uv, c8 = rest - g * uv;
        u32x4_t v = {0u, 0u, 0u, 0u};
        if (kin < live) v = gload<u32x4_t>(vbp + ((size_t)(kin * G + g) * DV + c8 * 8) * 2);
        *reinterpret_cast<u32x4_t*>(vsm + (g * 16 + kin) * pitchv + c8 * 16) = v;
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      const int h = wave + 8 * i;
      if (h < H) {
        const unsigned char* kt = ksm + ((h / hpg) * 16 + ni) * pitchk + kb * 16;
        f32x4_t sacc = z4;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          if (ks * 32 < D) sacc = mfma_bf16t(*reinterpret_cast<const u32x4_t*>(kt + ks * 64), qf[i][ks], sacc);
        float sv[4], mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = key0 + kb * 4 + r;
          const bool seen = key <= p && (a.window <= 0 || p - key < a.window);
          sv[r] = seen ? sacc[r] * mul[i] : -INFINITY;
          mx = fmaxf(mx, sv[r]);
        }
        if (PASS == 1) {
          mx = rows_max(mx);
          const float mn = fmaxf(mrun[i], mx);
          float ps = 0.f;
#pragma unroll
          for (int r = 0; r < 4; ++r) ps += __expf(sv[r] - mn);
          lrun[i] = lrun[i] * __expf(mrun[i] - mn) + rows_sum(ps);
          mrun[i] = mn;
        } else {
          const f32x4_t pv = {__expf(sv[0] - mrun[i]) * lrun[i], __expf(sv[1] - mrun[i]) * lrun[i], __expf(sv[2] - mrun[i]) * lrun[i],
                              __expf(sv[3] - mrun[i]) * lrun[i]};
          *reinterpret_cast<f32x4_t*>(psm + ((size_t)h * 16 + ni) * 16 + kb * 4) = pv;
        }
      }
    }
    if (PASS == 2) {
      __syncthreads();
      f32x4_t pm[OPW];
      int oh[OPW];
#pragma unroll
      for (int i = 0; i < OPW; ++i) { pm[i] = z4; oh[i] = (blockIdx.z * OPW + i) * 8 + wave; }
      if (oh[0] < H) {
        const float* pl = psm + ni * 16 + kb * 4;
        for (int g = 0; g < H; ++g) {
          const f32x4_t pv = *reinterpret_cast<const f32x4_t*>(pl + g * 256);
#pragma unroll
          for (int i = 0; i < OPW; ++i) {
            const float tw = oh[i] < H ? ((talk_uniform_ptr)(a.talk32))[oh[i] * H + g] : 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r) pm[i][r] = __builtin_fmaf(tw, pv[r], pm[i][r]);
          }
        }
#pragma unroll
        for (int i = 0; i < OPW; ++i) {
          if (oh[i] < H) {
            const u32x2_t pf = {pack_bf16x2(pm[i][0], pm[i][1]), pack_bf16x2(pm[i][2], pm[i][3])};
            const unsigned char* tr0 = vsm + ((oh[i] / hpg) * 16 + kb * 4 + (ni >> 2)) * pitchv + (ni & 3) * 8;
#pragma unroll
            for (int t = 0; t < DT; ++t)
              if (t * 16 < DV) oacc[i][t] = mfma_bf16k16(lds_read_tr16(tr0 + t * 32), pf, oacc[i][t]);
          }
        }
      }
    }
    __syncthreads();
  }
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
  if (!row_ok) return;
  if (PASS == 1) {
    if (kb == 0 && blockIdx.z == 0) {
#pragma unroll
      for (int i = 0; i < HPW; ++i) {
        const int h = wave + 8 * i;
        if (h < H) {
          float* st = a.stats + ((size_t)(row0 + tq) * H + h) * 2;
          st[0] = mrun[i];
          st[1] = lrun[i];
        }
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < OPW; ++i) {
    const int h = (blockIdx.z * OPW + i) * 8 + wave;
    if (h >= H) continue;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      if (t * 16 >= DV) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const size_t c = (size_t)h * DV + t * 16 + kb * 4 + r;
        const float v = oacc[i][t][r];
        st_any(a.out, (size_t)(row0 + tq) * a.ldo + c, a.odt, a.gate ? v * a.gate[(size_t)(row0 + tq) * a.ldg + c] : v);
      }
    }
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

/* Few rows (decoding): the same result with the work spread over (row, head, chunk) -- see talk_scores / talk_mix.  max_keys: a host
 * bound on the keys any row reads (min(window, last position + 1)).  Workspace: scores, statistics and parts. */
static int talk_few_chunks(int max_keys) { return (max_keys + 63) / 64; }
size_t dihip_talk_attn_few_workspace_bytes(int T, int H, int DV, int max_keys) {
  const int nchunk = talk_few_chunks(max_keys), nparts = (nchunk + 3) / 4;
  return ((size_t)T * H * nchunk * 64 + (size_t)T * nchunk * H * 2 + (nparts > 1 ? (size_t)T * nparts * H * DV : 0)) * sizeof(float);
}

int dihip_talk_attn_few(void* stream, void* out, int out_dtype, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                        int span_stride, int span_len, int cache_dtype, const void* temp, const void* talk, int w_dtype, const float* gate, long ldg,
                        const int32_t* tok_slot, const int32_t* tok_pos, int T, int H, int G, int D, int DV, float scale, int window, int max_keys,
                        void* ws, size_t ws_bytes) {
  DIHIP_REQUIRE(T >= 0 && out && q && kspans && vspans && talk && tok_slot && tok_pos && span_stride > 0 && span_len > 0 && H > 0 && G > 0 &&
                    H % G == 0 && D > 0 && DV > 0 && ldo >= (long)H * DV && ldq >= (long)H * D && (!gate || ldg >= (long)H * DV) && max_keys >= 1 &&
                    seq_dtype_ok(out_dtype) && seq_dtype_ok(cache_dtype) && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "talk_attn_few: bad argument");
  DIHIP_REQUIRE(H <= TALK_MAX_H && DV <= 256, DIHIP_EXCEED_LIMIT_ERROR, "talk_attn_few: at most %d heads and values of at most 256 elements", TALK_MAX_H);
  const int nchunk = talk_few_chunks(max_keys), nparts = (nchunk + 3) / 4;
  DIHIP_REQUIRE(nchunk <= 65535 && H <= 65535, DIHIP_PARAM_ERROR, "talk_attn_few: too many keys for one launch");
  DIHIP_REQUIRE(ws && ws_bytes >= dihip_talk_attn_few_workspace_bytes(T, H, DV, max_keys) && (reinterpret_cast<uintptr_t>(ws) & 3u) == 0,
                DIHIP_PARAM_ERROR, "talk_attn_few: workspace too small");
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  float* S = (float*)ws;
  float* stats = S + (size_t)T * H * nchunk * 64;
  TalkFewArgs f{TalkArgs{out, out_dtype, ldo, q, ldq, kspans, vspans, span_stride, span_len, temp, talk, w_dtype, gate, ldg, tok_slot, tok_pos,
                         H, G, D, DV, scale, window, nparts, stats, stats + (size_t)T * nchunk * H * 2},
                S, nchunk * 64, nchunk};
  auto go = [&](auto ct) {
    constexpr int CT = decltype(ct)::value;
    hipLaunchKernelGGL(talk_scores_kernel<CT>, dim3(T, H, nchunk), dim3(64), 0, s, f);
    if (DV <= 64) hipLaunchKernelGGL((talk_mix_kernel<CT, 1>), dim3(T, H, nparts), dim3(256), 0, s, f);
    else if (DV <= 128) hipLaunchKernelGGL((talk_mix_kernel<CT, 2>), dim3(T, H, nparts), dim3(256), 0, s, f);
    else hipLaunchKernelGGL((talk_mix_kernel<CT, 4>), dim3(T, H, nparts), dim3(256), 0, s, f);
  };
  if (cache_dtype == DIHIP_F32) go(std::integral_constant<int, DIHIP_F32>{});
  else go(std::integral_constant<int, DIHIP_BF16>{});
  if (nparts > 1) hipLaunchKernelGGL(talk_merge_kernel, dim3(T, T >= 256 ? 1 : (H * DV + 1023) / 1024), dim3(256), 0, s, f.a);
  return launch_status();
}

static size_t talk_mc_lds_bytes(int pass, int H, int G, int D, int DV) {
  size_t b = (size_t)G * 16 * (D + 8) * 2;
  if (pass == 2) b += (size_t)G * 16 * (DV + 8) * 2 + (size_t)H * 256 * sizeof(float);
  return b;
}

/* 1 when the matrix-core form serves these sizes on this device (bf16 pages) */
int dihip_talk_attn_mc_supported(int H, int G, int D, int DV, int span_len, int cache_dtype) {
  if (cache_dtype != DIHIP_BF16 || H < 1 || H > 32 || G < 1 || H % G || D % 32 || D > 128 || DV % 16 || DV > 128 || span_len % 16) return 0;
  return talk_mc_lds_bytes(2, H, G, D, DV) <= 160 * 1024 - 1024;
}

size_t dihip_talk_attn_mc_workspace_bytes(int T, int H) { return (size_t)T * H * 2 * sizeof(float); }

int dihip_talk_attn_mc(void* stream, void* out, int out_dtype, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                       int span_stride, int span_len, const void* temp, int w_dtype, const float* talk32, const float* gate, long ldg,
                       const int32_t* tok_pos, const int32_t* ent_slot, const int32_t* ent_row0, const int32_t* ent_count, int E, int max_count,
                       int T, int H, int G, int D, int DV, float scale, int window, void* ws, size_t ws_bytes) {
  DIHIP_REQUIRE(T >= 0 && E >= 0 && max_count >= 0 && out && q && kspans && vspans && talk32 && tok_pos && ent_slot && ent_row0 && ent_count &&
                    span_stride > 0 && span_len > 0 && ldo >= (long)H * DV && ldq >= (long)H * D && (!gate || ldg >= (long)H * DV) &&
                    seq_dtype_ok(out_dtype) && seq_dtype_ok(w_dtype) && E <= 65535, DIHIP_PARAM_ERROR, "talk_attn_mc: bad argument");
  DIHIP_REQUIRE(dihip_talk_attn_mc_supported(H, G, D, DV, span_len, DIHIP_BF16), DIHIP_EXCEED_LIMIT_ERROR,
                "talk_attn_mc: sizes the matrix-core form does not serve (H <= 32, D %% 32 == 0 <= 128, DV %% 16 == 0 <= 128)");
  DIHIP_REQUIRE((ldq & 3) == 0 && (reinterpret_cast<uintptr_t>(q) & 15u) == 0, DIHIP_PARAM_ERROR, "talk_attn_mc: query rows must be 16-byte aligned");
  DIHIP_REQUIRE(ws && ws_bytes >= dihip_talk_attn_mc_workspace_bytes(T, H) && (reinterpret_cast<uintptr_t>(ws) & 3u) == 0, DIHIP_PARAM_ERROR,
                "talk_attn_mc: workspace too small");
  if (T == 0 || E == 0 || max_count == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  TalkMcArgs a{out, out_dtype, ldo, q, ldq, kspans, vspans, span_stride, span_len, temp, w_dtype, talk32, gate, ldg, tok_pos, ent_slot, ent_row0,
               ent_count, H, G, D, DV, scale, window, (float*)ws};
  const int tiles = (max_count + 15) / 16;
  const size_t lds1 = talk_mc_lds_bytes(1, H, G, D, DV), lds2 = talk_mc_lds_bytes(2, H, G, D, DV);
  int status = DIHIP_SUCCESS;
  auto go = [&](auto hpw, auto opw, auto dmax, auto vmax) {
    constexpr int HPW = decltype(hpw)::value, OPW = decltype(opw)::value, DMAX = decltype(dmax)::value, VMAX = decltype(vmax)::value;
    auto k1 = talk_attn_mc_kernel<1, HPW, 1, DMAX, 16>;
    auto k2 = talk_attn_mc_kernel<2, HPW, OPW, DMAX, VMAX>;
    if (lds1 > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(k1), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds1) != hipSuccess) status = DIHIP_RUNTIME_ERROR;
    if (lds2 > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(k2), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds2) != hipSuccess) status = DIHIP_RUNTIME_ERROR;
    if (status != DIHIP_SUCCESS) { (void)hipGetLastError(); return; }
    hipLaunchKernelGGL(k1, dim3(tiles, E, 1), dim3(512), lds1, s, a);
    hipLaunchKernelGGL(k2, dim3(tiles, E, HPW / OPW), dim3(512), lds2, s, a);
  };
  auto by_size = [&](auto hpw, auto opw) {
    using d64 = std::integral_constant<int, 64>;
    using d128 = std::integral_constant<int, 128>;
    if (D <= 64) { if (DV <= 64) go(hpw, opw, d64{}, d64{}); else go(hpw, opw, d64{}, d128{}); }
    else { if (DV <= 64) go(hpw, opw, d128{}, d64{}); else go(hpw, opw, d128{}, d128{}); }
  };
  using c1 = std::integral_constant<int, 1>;
  using c2 = std::integral_constant<int, 2>;
  using c4 = std::integral_constant<int, 4>;
  if (H <= 8) by_size(c1{}, c1{});
  else if (H <= 16) by_size(c2{}, c2{});
  else by_size(c4{}, c2{});
  DIHIP_REQUIRE(status == DIHIP_SUCCESS, DIHIP_RUNTIME_ERROR, "talk_attn_mc: the device refused %zu bytes of LDS for a workgroup", lds2);
  return launch_status();
}

}  // extern "C"
