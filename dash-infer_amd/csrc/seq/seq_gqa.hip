// seq_gqa.hip -- grouped-query attention over paged key and value caches for the sequence engine:
//   qkv_prep_append   per token: unit-RMS norm of every query / key head (optional), rotary positions (paired or half-split
//                     layout, a frequency table and a magnitude from the host), mixing of the values with another layer's,
//                     queries written back in place, keys and values appended to their pages
//   gqa_attn_kernel   one workgroup per row, every product and sum in f32 (any cache type)
//   gqa_attn_mc_kernel + merge   bf16 caches on the matrix cores, the key walk split for few rows (decoding)
// Options of the softmax: a sink logit per head or the constant 0 (one more term in the denominator, no value), a tanh cap on
// the scores, a multiplier per (row, head) on the output (the output gate).
// Options of the key walk: a sliding window with kept first keys (row p reads key j <= p if p - j < window or j < keep_first;
// the keys between are skipped by whole chunks / tiles), and several softmax maps per head (`maps`: head h has maps query
// vectors and its key head maps key vectors, laid out one after the other; map m of a head scores against map m of its key
// head, all maps read the same values; the output holds the maps of a head side by side).
//   maps_diff_norm    two maps per head -> one: (first - lam * second) / its root mean square * a constant
#include "seq_common.h"

namespace dihip {
namespace {

// ------------------------------------------------------------------------------------------------ prep + append
struct PrepArgs {
  float* qkv; long ld; int q_off, k_off, v_off;
  int H, G, D, DV, GV;   // H / G: query / key vectors per token (heads x maps), GV: value heads
  const void* qnorm; const void* knorm; int wdt; float eps;
  const float* freq; int rot_dims, layout; float mag;
  float lam; const float* vfirst_in; float* vfirst_out; long ldvf;
  void* const* kspans; void* const* vspans; int span_stride, span_len, cdt;
  const int32_t* tok_slot; const int32_t* tok_pos;
};

__global__ __launch_bounds__(256) void qkv_prep_append_kernel(PrepArgs a) {
  __shared__ float hs[4][256];
  __shared__ float cs_t[128], sn_t[128];   // the token's cos and sin per rotated pair, shared by all heads
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pos = a.tok_pos[t];
  if (threadIdx.x < (a.rot_dims >> 1)) {
    float sn, cs;
    rope_sincos((uint32_t)pos, a.freq[threadIdx.x], &sn, &cs);
    cs_t[threadIdx.x] = cs * a.mag;
    sn_t[threadIdx.x] = sn * a.mag;
  }
  const size_t sp = (size_t)a.tok_slot[t] * a.span_stride + pos / a.span_len;
  const size_t in_span = (size_t)(pos % a.span_len);
  float* row = a.qkv + (size_t)t * a.ld;
  const int D = a.D, half = a.rot_dims >> 1;
  for (int h0 = blockIdx.y * 4; h0 < a.H + a.G; h0 += 4 * gridDim.y) {      // query heads, then key heads: the same trip count in every wave
    const int hh = h0 + wave;
    const bool live = hh < a.H + a.G, is_q = hh < a.H;
    float* src = row + (is_q ? a.q_off + hh * D : a.k_off + (hh - a.H) * D);
    const void* gamma = is_q ? a.qnorm : a.knorm;
    float v[4], ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      v[i] = live && d < D ? src[d] : 0.f;
      ss = __builtin_fmaf(v[i], v[i], ss);
    }
    if (gamma) {
      const float inv = 1.f / sqrtf(wave_sum(ss) / (float)D + a.eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = lane + 64 * i;
        if (d < D) v[i] = v[i] * inv * ld_any(gamma, d, a.wdt);
      }
    }
    __syncthreads();   // hs of the head before is no longer read
#pragma unroll
    for (int i = 0; i < 4; ++i) hs[wave][lane + 64 * i] = v[i];
    __syncthreads();
    if (live) {
      void* kdst = is_q ? nullptr : a.kspans[sp];
      const size_t kbase = (in_span * a.G + (size_t)(is_q ? 0 : hh - a.H)) * D;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = lane + 64 * i;
        if (d >= D) continue;
        float y = v[i];
        if (d < a.rot_dims) {
          int pair, other;
          bool first;
          if (a.layout == 0) { pair = d >> 1; first = (d & 1) == 0; other = d ^ 1; }
          else { first = d < half; pair = first ? d : d - half; other = first ? d + half : d - half; }
          const float sn = sn_t[pair], cs = cs_t[pair];
          const float o = hs[wave][other];
          y = first ? v[i] * cs - o * sn : v[i] * cs + o * sn;
        }
        if (is_q) src[d] = y;
        else st_any(kdst, kbase + d, a.cdt, y);
      }
    }
  }
  void* vdst = a.vspans[sp];
  const int nv = a.GV * a.DV;
  for (int e = blockIdx.y * 256 + threadIdx.x; e < nv; e += 256 * gridDim.y) {
    float v = row[a.v_off + e];
    if (a.vfirst_in) v = (1.f - a.lam) * v + a.lam * a.vfirst_in[(size_t)t * a.ldvf + e];
    if (a.vfirst_out) a.vfirst_out[(size_t)t * a.ldvf + e] = v;
    st_any(vdst, in_span * nv + e, a.cdt, v);
  }
}

// ------------------------------------------------------------------------------------------------ f32 row kernel
struct GqaArgs {
  float* out; long ldo;
  const float* q; long ldq;
  void* const* kspans; void* const* vspans; int span_stride, span_len;
  const void* sink; int wdt, sink_mode;   // 0: none, 1: sink[h], 2: the constant 0
  float softcap;                          // <= 0: none
  const float* gate; long ldg;            // [T, H] multiplier (NULL: none)
  const int32_t* tok_slot; const int32_t* tok_pos; const int32_t* ent_slot; const int32_t* ent_row0; const int32_t* ent_count;
  int H, G, D, DV; float scale;
  float* ws; int rows_total;
  int maps, window, keep_first;           // window <= 0: every key up to the row's own
};

__device__ __forceinline__ float cap_score(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

// One workgroup per row, its 4 waves take the (head, map) pairs in turn; a wave walks the keys it may read 64 at a time (first the
// kept first keys that lie before the window, then the window): lane j scores key j (d ascending), the chunk joins the running
// softmax, then the lanes turn to the value elements and add the weighted rows.
template <int CT, int RV>
__global__ __launch_bounds__(256) void gqa_attn_kernel(GqaArgs a) {
  __shared__ float qs[4][256];
  __shared__ float ps[4][64];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pos = a.tok_pos[t], H = a.H, G = a.G, D = a.D, DV = a.DV, hpg = H / G, M = a.maps, HQ = H * M, GK = G * M;
  const int w_lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;   // the window is [w_lo, pos]
  const int first_hi = min(a.keep_first, w_lo);                     // the kept first keys before it: [0, first_hi)
  void* const* ktab = a.kspans + (size_t)a.tok_slot[t] * a.span_stride;
  void* const* vtab = a.vspans + (size_t)a.tok_slot[t] * a.span_stride;
  constexpr size_t ES = CT == DIHIP_F32 ? 4 : 2;
  for (int h0 = 0; h0 < HQ; h0 += 4) {
    const int hq = h0 + wave;
    const bool live = hq < HQ;
    const int h = (live ? hq : 0) / M, mp = (live ? hq : 0) - h * M;
    const int g = h / hpg, gk = g * M + mp;
    __syncthreads();
    if (live)
      for (int d = lane; d < D; d += 64) qs[wave][d] = a.q[(size_t)t * a.ldq + (size_t)hq * D + d];
    __syncthreads();
    float mx = -INFINITY, den = 0.f;
    if (a.sink_mode == 1) { mx = ld_any(a.sink, h, a.wdt); den = 1.f; }
    else if (a.sink_mode == 2) { mx = 0.f; den = 1.f; }
    float acc[RV];
#pragma unroll
    for (int v = 0; v < RV; ++v) acc[v] = 0.f;
    for (int part = 0; part < 2; ++part) {                       // the same trip counts in every wave of the block
      const int r_lo = part ? w_lo : 0, r_hi = part ? pos + 1 : first_hi;
      for (int j0 = r_lo; j0 < r_hi; j0 += 64) {
        const int j = j0 + lane;
        const bool valid = live && j < r_hi;
        float s = -INFINITY;
        if (valid) {
          const char* kr = (const char*)ktab[j / a.span_len] + ((size_t)(j % a.span_len) * GK + gk) * D * ES;
          float d = 0.f;
          for (int r = 0; r < D; ++r) d = __builtin_fmaf(qs[wave][r], load_ft<CT>(kr, r), d);
          s = cap_score(d * a.scale, a.softcap);
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
          const int cnt = min(64, r_hi - j0);
          for (int jj = 0; jj < cnt; ++jj) {
            const int jk = j0 + jj;
            const char* vr = (const char*)vtab[jk / a.span_len] + ((size_t)(jk % a.span_len) * G + g) * DV * ES;
            const float pj = ps[wave][jj];
#pragma unroll
            for (int v = 0; v < RV; ++v) {
              const int r = v * 64 + lane;
              if (r < DV) acc[v] = __builtin_fmaf(pj, load_ft<CT>(vr, r), acc[v]);
            }
          }
        }
        __syncthreads();
      }
    }
    if (live) {
      const float gt = a.gate ? a.gate[(size_t)t * a.ldg + h] : 1.f;
#pragma unroll
      for (int v = 0; v < RV; ++v) {
        const int r = v * 64 + lane;
        if (r < DV) a.out[(size_t)t * a.ldo + (size_t)hq * DV + r] = acc[v] / den * gt;
      }
    }
  }
}

// Two maps per head -> one: d = first - lam * second, out = d / sqrt(mean(d^2) + eps) * out_scale.  A wave per (row, head).
__global__ __launch_bounds__(256) void maps_diff_norm_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ x, long ldx,
                                                             float lam, float out_scale, float eps, int TH, int H, int DV) {
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (pair >= TH) return;
  const int t = pair / H, h = pair - t * H;
  const float* a1 = x + (size_t)t * ldx + (size_t)h * 2 * DV;
  const float* a2 = a1 + DV;
  float v[8], ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + 64 * i;
    v[i] = d < DV ? a1[d] - lam * a2[d] : 0.f;
    ss = __builtin_fmaf(v[i], v[i], ss);
  }
  const float inv = out_scale / sqrtf(wave_sum(ss) / (float)DV + eps);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + 64 * i;
    if (d < DV) st_any(y, (size_t)t * ldy + (size_t)h * DV + d, ydt, v[i] * inv);
  }
}

// ------------------------------------------------------------------------------------------------ matrix-core kernel
// A workgroup owns 64 consecutive (row, query head) pairs of ONE portion, ONE key/value head and ONE map -- 16 per wave -- and
// walks the 32-key tiles those pairs can see (with a window: the tiles of the kept first keys, then those from the window of its
// first row on).  Per tile: S^T = K . Q^T (the tile's key rows as they lie in LDS against the wave's
// query fragments, held in registers for the whole walk), cap + mask + running softmax on the accumulator lanes, then
// O^T += V^T . P^T with P straight from those lanes and V^T read from the value tile through the transposing LDS read.  The
// next tile's rows are in flight meanwhile.  Head sizes that are no multiple of the tile's granule are padded with zero
// columns in LDS.  The key walk can be split over gridDim.z workgroups; the partial records are merged by a second launch.
__device__ __forceinline__ f32x4_t mfma_bf16g(const u32x4_t& a, const u32x4_t& b, const f32x4_t& c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ float fast_tanh(float x) { return 1.f - 2.f / (1.f + __expf(2.f * x)); }

template <int DMAX, int VMAX>
__global__ __launch_bounds__(256) void gqa_attn_mc_kernel(GqaArgs a) {
  constexpr int KS = DMAX / 32, DT = VMAX / 16, UNK = DMAX / 64, UNV = VMAX / 64;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int G = a.G, H = a.H, D = a.D, DV = a.DV, hpg = H / G;
  const int M = a.maps, GK = G * M;
  const int e = blockIdx.y / GK, gk = blockIdx.y - e * GK, g = gk / M, mp = gk - g * M, split = blockIdx.z, nsplit = gridDim.z;
  const int cnt = a.ent_count[e], row0 = a.ent_row0[e];
  const int nrows = cnt * hpg, r0 = blockIdx.x * 64;
  if (r0 >= nrows) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, ni = lane & 15, kb = lane >> 4;
  const int Dp = (D + 31) & ~31, Vp = (DV + 15) & ~15;
  const int pitchk = (Dp + 8) * 2, pitchv = (Vp + 8) * 2;
  unsigned char* ksm = smem;
  unsigned char* vsm = smem + 32 * pitchk;
  const int pos0 = a.tok_pos[row0];
  const int myrow = r0 + wave * 16 + ni;
  const bool row_ok = myrow < nrows;
  const int rr = row_ok ? myrow : nrows - 1;
  const int tq = rr / hpg, h = g * hpg + (rr - tq * hpg), hq = h * M + mp, p = pos0 + tq;
  const int p_lo = pos0 + r0 / hpg, p_hi = pos0 + min(r0 + 63, nrows - 1) / hpg;
  const int tile_hi = p_hi >> 5;
  const int win_t0 = (a.window > 0 ? max(0, p_lo - a.window + 1) : 0) >> 5;          // the first tile of the window of the first row
  const int n_first = min(win_t0, (min(a.keep_first, p_hi + 1) + 31) >> 5);           // tiles of kept first keys before it
  const int n_tiles = n_first + tile_hi - win_t0 + 1;
  const int per = (n_tiles + nsplit - 1) / nsplit;
  const int my_lo = split * per, my_hi = min(n_tiles - 1, my_lo + per - 1);           // indices into the walk: tile_of(i)
  auto tile_of = [&](int i) { return i < n_first ? i : win_t0 + (i - n_first); };

  u32x4_t qf[KS];
  {
    const float* qrow = a.q + (size_t)(row0 + tq) * a.ldq + (size_t)hq * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = u32x4_t{0u, 0u, 0u, 0u};
      const int d0 = ks * 32 + kb * 8;
      if (d0 < D) {   // D % 8 == 0: a unit of 8 is inside or outside
        const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(qrow + d0);
        const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(qrow + d0 + 4);
        qf[ks] = u32x4_t{pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3])};
      }
    }
  }
  const bool with_sink = a.sink_mode != 0 && split == 0;
  float m = with_sink ? (a.sink_mode == 1 ? ld_any(a.sink, h, a.wdt) : 0.f) : -1e30f;
  float l = with_sink ? 1.f : 0.f;
  const f32x4_t z4 = {0.f, 0.f, 0.f, 0.f};
  f32x4_t oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) oacc[t] = z4;

  // zero the padding columns once: the tiles' stores never touch them
  for (int i = tid; i < 32 * (Dp - D + 8); i += 256) {
    const int kin = i / (Dp - D + 8), c = D + i % (Dp - D + 8);
    reinterpret_cast<uint16_t*>(ksm + kin * pitchk)[c] = 0;
  }
  for (int i = tid; i < 32 * (Vp - DV + 8); i += 256) {
    const int kin = i / (Vp - DV + 8), c = DV + i % (Vp - DV + 8);
    reinterpret_cast<uint16_t*>(vsm + kin * pitchv)[c] = 0;
  }
  __shared__ const char* ktabs[128];
  __shared__ const char* vtabs[128];
  void* const* gkp = a.kspans + (size_t)a.ent_slot[e] * a.span_stride;
  void* const* gv = a.vspans + (size_t)a.ent_slot[e] * a.span_stride;
  const int span_lo = my_lo <= my_hi ? (tile_of(my_lo) * 32) / a.span_len : 0;
  for (int i = tid; i < 128; i += 256) {
    const int sp = span_lo + i;
    const bool in = sp * a.span_len <= p_hi;
    ktabs[i] = in ? (const char*)gkp[sp] : nullptr;
    vtabs[i] = in ? (const char*)gv[sp] : nullptr;
  }
  __syncthreads();
  const int uprk = D >> 3, uprv = DV >> 3;
  int gok[UNK], lok[UNK], gov[UNV], lov[UNV];
#pragma unroll
  for (int j = 0; j < UNK; ++j) {
    const int u = tid + 256 * j, kin = u / uprk, c8 = u - kin * uprk;
    gok[j] = kin < 32 ? ((kin * GK + gk) * D + c8 * 8) * 2 : -1;
    lok[j] = kin * pitchk + c8 * 16;
  }
#pragma unroll
  for (int j = 0; j < UNV; ++j) {
    const int u = tid + 256 * j, kin = u / uprv, c8 = u - kin * uprv;
    gov[j] = kin < 32 ? ((kin * G + g) * DV + c8 * 8) * 2 : -1;
    lov[j] = kin * pitchv + c8 * 16;
  }
  u32x4_t prek[UNK], prev[UNV];
  auto fetch = [&](int tile) {
    const int key0 = tile * 32, sp = key0 / a.span_len, in = key0 - sp * a.span_len;
    const bool near = sp - span_lo < 128;
    const char* kbp = (near ? ktabs[sp - span_lo] : (const char*)gkp[sp]) + (size_t)in * GK * D * 2;
    const char* vbp = (near ? vtabs[sp - span_lo] : (const char*)gv[sp]) + (size_t)in * G * DV * 2;
#pragma unroll
    for (int j = 0; j < UNK; ++j) {
      prek[j] = u32x4_t{0u, 0u, 0u, 0u};
      if (gok[j] >= 0) prek[j] = gload<u32x4_t>(kbp + gok[j]);
    }
#pragma unroll
    for (int j = 0; j < UNV; ++j) {
      prev[j] = u32x4_t{0u, 0u, 0u, 0u};
      if (gov[j] >= 0) prev[j] = gload<u32x4_t>(vbp + gov[j]);
    }
  };
  if (my_lo <= my_hi) fetch(tile_of(my_lo));
  for (int ti = my_lo; ti <= my_hi; ++ti) {
    const int tile = tile_of(ti);
#pragma unroll
    for (int j = 0; j < UNK; ++j)
      if (gok[j] >= 0) *reinterpret_cast<u32x4_t*>(ksm + lok[j]) = prek[j];
#pragma unroll
    for (int j = 0; j < UNV; ++j)
      if (gov[j] >= 0) *reinterpret_cast<u32x4_t*>(vsm + lov[j]) = prev[j];
    __syncthreads();
    if (ti + 1 <= my_hi) fetch(tile_of(ti + 1));
    f32x4_t sacc[2] = {z4, z4};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks * 32 < D) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          const u32x4_t kf = *reinterpret_cast<const u32x4_t*>(ksm + (nt * 16 + ni) * pitchk + (ks * 32 + kb * 8) * 2);
          sacc[nt] = mfma_bf16g(kf, qf[ks], sacc[nt]);
        }
      }
    }
    float sv[2][4], mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = tile * 32 + nt * 16 + kb * 4 + r;
        float s = sacc[nt][r] * a.scale;
        if (a.softcap > 0.f) s = a.softcap * fast_tanh(s / a.softcap);
        const bool seen = key <= p && (a.window <= 0 || p - key < a.window || key < a.keep_first);
        sv[nt][r] = seen ? s : -INFINITY;
        mx = fmaxf(mx, sv[nt][r]);
      }
    mx = rows_max(mx);
    const float mn = fmaxf(m, mx);
    const float corr = __expf(m - mn);
    m = mn;
    float psum = 0.f, ev[2][4];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        ev[nt][r] = __expf(sv[nt][r] - mn);
        psum += ev[nt][r];
      }
    l = l * corr + rows_sum(psum);
    const u32x4_t pf = {pack_bf16x2(ev[0][0], ev[0][1]), pack_bf16x2(ev[0][2], ev[0][3]), pack_bf16x2(ev[1][0], ev[1][1]),
                        pack_bf16x2(ev[1][2], ev[1][3])};
    if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0ull) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) oacc[t][r] *= corr;
    }
    const unsigned char* tr0 = vsm + (kb * 4 + (ni >> 2)) * pitchv + (ni & 3) * 8;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      if (t * 16 < DV) {
        const u32x2_t lo2 = lds_read_tr16(tr0 + t * 32);
        const u32x2_t hi2 = lds_read_tr16(tr0 + t * 32 + 16 * pitchv);
        const u32x4_t vf = {lo2[0], lo2[1], hi2[0], hi2[1]};
        oacc[t] = mfma_bf16g(vf, pf, oacc[t]);
      }
    }
    __syncthreads();
  }
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
  if (!row_ok) return;
  if (nsplit == 1) {
    const float inv = (a.gate ? a.gate[(size_t)(row0 + tq) * a.ldg + h] : 1.f) / l;
    float* o = a.out + (size_t)(row0 + tq) * a.ldo + (size_t)hq * DV + kb * 4;
#pragma unroll
    for (int t = 0; t < DT; ++t)
      if (t * 16 + kb * 4 < DV) *reinterpret_cast<f32x4_t*>(o + t * 16) = f32x4_t{oacc[t][0] * inv, oacc[t][1] * inv, oacc[t][2] * inv, oacc[t][3] * inv};
  } else {
    float* o = a.ws + ((size_t)split * a.rows_total + (size_t)(row0 + tq) * H * M + hq) * (Vp + 4);
#pragma unroll
    for (int t = 0; t < DT; ++t)
      if (t * 16 < Vp) *reinterpret_cast<f32x4_t*>(o + t * 16 + kb * 4) = oacc[t];
    if (kb == 0) { o[Vp] = m; o[Vp + 1] = l; }
  }
}

// The splits' (maximum, denominator, sums) records of one (row, query vector) -> column threadIdx.x of its softmax-weighted sum
// (0 for threads past DV; DV <= 256).  wgt / red: LDS scratch of the workgroup; the call synchronises it.
__device__ __forceinline__ float merge_splits(const float* __restrict__ base, size_t stride, int nsplit, int Vp, int DV, float* wgt, float* red) {
  float mloc[4], lloc[4], mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int s = threadIdx.x + i * 256;
    mloc[i] = s < nsplit ? base[s * stride + Vp] : -INFINITY;
    lloc[i] = s < nsplit ? base[s * stride + Vp + 1] : 0.f;
    mx = fmaxf(mx, mloc[i]);
  }
  mx = wave_max(mx);
  __syncthreads();                   // wgt / red of an earlier call are no longer read
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float den = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int s = threadIdx.x + i * 256;
    const float w = s < nsplit ? expf(mloc[i] - mx) : 0.f;
    if (s < nsplit) wgt[s] = w;
    den = __builtin_fmaf(w, lloc[i], den);
  }
  den = block256_sum(den, red);      // (its barriers publish wgt)
  float acc = 0.f;
  const int r = threadIdx.x;
  if (r < DV) {
#pragma unroll 8
    for (int s = 0; s < nsplit; ++s) acc = __builtin_fmaf(wgt[s], base[s * stride + r], acc);
  }
  return acc / den;
}

// one workgroup per (row, query vector)
__global__ __launch_bounds__(256) void gqa_attn_merge_kernel(float* __restrict__ out, long ldo, const float* __restrict__ ws, int nsplit,
                                                             int rows_total, int H, int maps, int DV, int Vp, const float* __restrict__ gate, long ldg) {
  __shared__ float wgt[1024];
  __shared__ float red[4];
  const int gi = blockIdx.x, HQ = H * maps, t = gi / HQ, hq = gi - t * HQ, h = hq / maps;
  const size_t rec = (size_t)Vp + 4;
  const float v = merge_splits(ws + (size_t)gi * rec, (size_t)rows_total * rec, nsplit, Vp, DV, wgt, red);
  if (threadIdx.x < DV) out[(size_t)t * ldo + (size_t)hq * DV + threadIdx.x] = v * (gate ? gate[(size_t)t * ldg + h] : 1.f);
}

// one workgroup per (row, head) of two maps: both merged, then d = first - lam * second, y = d / sqrt(mean(d^2) + eps) * out_scale
__global__ __launch_bounds__(256) void gqa_attn_merge_diff_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ ws, int nsplit,
                                                                  int rows_total, int H, int DV, int Vp, const float* __restrict__ gate, long ldg,
                                                                  float lam, float out_scale, float eps) {
  __shared__ float wgt[1024];
  __shared__ float red[4];
  const int gi = blockIdx.x, t = gi / H, h = gi - t * H;
  const size_t rec = (size_t)Vp + 4, stride = (size_t)rows_total * rec;
  const float* base = ws + ((size_t)t * H * 2 + (size_t)h * 2) * rec;
  const float a1 = merge_splits(base, stride, nsplit, Vp, DV, wgt, red);
  const float a2 = merge_splits(base + rec, stride, nsplit, Vp, DV, wgt, red);
  const float d = (a1 - lam * a2) * (gate ? gate[(size_t)t * ldg + h] : 1.f);
  const float inv = out_scale / sqrtf(block256_sum(d * d, red) / (float)DV + eps);
  if (threadIdx.x < DV) st_any(y, (size_t)t * ldy + (size_t)h * DV + threadIdx.x, ydt, d * inv);
}

}  // namespace
}  // namespace dihip

using namespace dihip;

extern "C" {

int dihip_qkv_prep_append(void* stream, float* qkv, long ld, int q_off, int k_off, int v_off, int H, int G, int D, int DV, int maps,
                          const void* qnorm, const void* knorm, int w_dtype, float eps, const float* freq, int rot_dims, int layout,
                          float mag, float lam, const float* vfirst_in, float* vfirst_out, long ldvf, void* const* kspans,
                          void* const* vspans, int span_stride, int span_len, int cache_dtype, const int32_t* tok_slot,
                          const int32_t* tok_pos, int T) {
  DIHIP_REQUIRE(T >= 0 && qkv && H > 0 && G > 0 && H % G == 0 && D > 0 && D <= 256 && DV > 0 && kspans && vspans && tok_slot && tok_pos &&
                    span_stride > 0 && span_len > 0 && seq_dtype_ok(cache_dtype) && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR,
                "qkv_prep_append: bad argument (heads of at most 256 elements)");
  DIHIP_REQUIRE(maps >= 1 && maps <= 8, DIHIP_PARAM_ERROR, "qkv_prep_append: 1 to 8 maps per head");
  const int GV = G;
  H *= maps;     // from here on: query / key vectors per token
  G *= maps;
  DIHIP_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && ld >= (long)q_off + (long)H * D && ld >= (long)k_off + (long)G * D &&
                    ld >= (long)v_off + (long)GV * DV, DIHIP_PARAM_ERROR, "qkv_prep_append: columns outside the rows");
  DIHIP_REQUIRE(rot_dims >= 0 && rot_dims <= D && rot_dims % 2 == 0 && (rot_dims == 0 || freq) && (layout == 0 || layout == 1),
                DIHIP_PARAM_ERROR, "qkv_prep_append: bad rotation (an even number of dimensions up to the head size, layout 0 / 1)");
  DIHIP_REQUIRE((!vfirst_in && !vfirst_out) || ldvf >= (long)GV * DV, DIHIP_PARAM_ERROR, "qkv_prep_append: value rows shorter than the values");
  if (T == 0) return DIHIP_SUCCESS;
  PrepArgs a{qkv, ld, q_off, k_off, v_off, H, G, D, DV, GV, qnorm, knorm, w_dtype, eps, freq, rot_dims, layout, mag, lam, vfirst_in, vfirst_out,
             ldvf, kspans, vspans, span_stride, span_len, cache_dtype, tok_slot, tok_pos};
  // few rows (decoding): the heads of a token are spread over workgroups of four; many rows: a workgroup per token
  hipLaunchKernelGGL(qkv_prep_append_kernel, dim3(T, T >= 256 ? 1 : (H + G + 3) / 4), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), a);
  return launch_status();
}

static int gqa_check(const char* what, const float* out, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                     int span_stride, int span_len, const void* sink, int w_dtype, int sink_mode, const float* gate, long ldg, int H, int G,
                     int D, int DV, int maps, int keep_first) {
  DIHIP_REQUIRE(maps >= 1 && maps <= 8 && keep_first >= 0, DIHIP_PARAM_ERROR, "%s: 1 to 8 maps per head, no negative count of kept keys", what);
  DIHIP_REQUIRE(out && q && kspans && vspans && span_stride > 0 && span_len > 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && DV > 0 &&
                    ldo >= (long)H * maps * DV && ldq >= (long)H * maps * D && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "%s: bad argument", what);
  DIHIP_REQUIRE(sink_mode >= 0 && sink_mode <= 2 && (sink_mode != 1 || sink) && (!gate || ldg >= H), DIHIP_PARAM_ERROR,
                "%s: bad sink mode or gate", what);
  return DIHIP_SUCCESS;
}

int dihip_gqa_attn(void* stream, float* out, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                   int span_stride, int span_len, int cache_dtype, const void* sink, int w_dtype, int sink_mode, float softcap,
                   const float* gate, long ldg, const int32_t* tok_slot, const int32_t* tok_pos, int T, int H, int G, int D, int DV,
                   float scale, int maps, int window, int keep_first) {
  if (int rc = gqa_check("gqa_attn", out, ldo, q, ldq, kspans, vspans, span_stride, span_len, sink, w_dtype, sink_mode, gate, ldg, H, G, D, DV, maps, keep_first)) return rc;
  DIHIP_REQUIRE(T >= 0 && tok_slot && tok_pos && seq_dtype_ok(cache_dtype), DIHIP_PARAM_ERROR, "gqa_attn: bad argument");
  DIHIP_REQUIRE(D <= 256 && DV <= 512, DIHIP_EXCEED_LIMIT_ERROR, "gqa_attn: head sizes above 256 (keys) / 512 (values)");
  if (T == 0) return DIHIP_SUCCESS;
  GqaArgs a{out, ldo, q, ldq, kspans, vspans, span_stride, span_len, sink, w_dtype, sink_mode, softcap, gate, ldg, tok_slot, tok_pos,
            nullptr, nullptr, nullptr, H, G, D, DV, scale, nullptr, 0, maps, window, keep_first};
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  auto go = [&](auto ct, auto rv) {
    constexpr int CT = decltype(ct)::value, RV = decltype(rv)::value;
    hipLaunchKernelGGL((gqa_attn_kernel<CT, RV>), dim3(T), dim3(256), 0, s, a);
  };
  auto by_v = [&](auto ct) {
    if (DV <= 64) go(ct, std::integral_constant<int, 1>{});
    else if (DV <= 128) go(ct, std::integral_constant<int, 2>{});
    else if (DV <= 256) go(ct, std::integral_constant<int, 4>{});
    else go(ct, std::integral_constant<int, 8>{});
  };
  if (cache_dtype == DIHIP_F32) by_v(std::integral_constant<int, DIHIP_F32>{});
  else by_v(std::integral_constant<int, DIHIP_BF16>{});
  return launch_status();
}

int dihip_gqa_attn_mc_supported(int D, int DV, int span_len, int cache_dtype) {
  return cache_dtype == DIHIP_BF16 && D % 8 == 0 && DV % 8 == 0 && D >= 8 && DV >= 8 && D <= 256 && DV <= 128 && span_len % 32 == 0;
}

size_t dihip_gqa_attn_mc_workspace_bytes(int T, int HQ, int DV, int nsplit) {
  return nsplit > 1 ? (size_t)nsplit * T * HQ * (((DV + 15) & ~15) + 4) * sizeof(float) : 0;
}

int dihip_gqa_attn_mc(void* stream, float* out, long ldo, const float* q, long ldq, void* const* kspans, void* const* vspans,
                      int span_stride, int span_len, const void* sink, int w_dtype, int sink_mode, float softcap, const float* gate,
                      long ldg, const int32_t* tok_pos, const int32_t* ent_slot, const int32_t* ent_row0, const int32_t* ent_count, int E,
                      int max_count, int T, int H, int G, int D, int DV, float scale, int maps, int window, int keep_first, int nsplit,
                      void* ws, size_t ws_bytes, void* diff_out, int diff_dtype, long ldd, float lam, float out_scale, float eps) {
  if (int rc = gqa_check("gqa_attn_mc", out, ldo, q, ldq, kspans, vspans, span_stride, span_len, sink, w_dtype, sink_mode, gate, ldg, H, G, D, DV, maps, keep_first)) return rc;
  DIHIP_REQUIRE(dihip_gqa_attn_mc_supported(D, DV, span_len, DIHIP_BF16), DIHIP_PARAM_ERROR,
                "gqa_attn_mc: head sizes %d / %d (multiples of 8 up to 256 / 128) or span_len %d (a multiple of 32) not served", D, DV, span_len);
  DIHIP_REQUIRE(E >= 0 && T >= 0 && max_count >= 0 && tok_pos && ent_slot && ent_row0 && ent_count && ldo % 4 == 0 && ldq % 4 == 0,
                DIHIP_PARAM_ERROR, "gqa_attn_mc: bad argument");
  DIHIP_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15u) == 0 && (reinterpret_cast<uintptr_t>(q) & 15u) == 0, DIHIP_PARAM_ERROR,
                "gqa_attn_mc: q / out must be 16-byte aligned");
  DIHIP_REQUIRE(nsplit >= 1 && nsplit <= 1024 && (long)E * G * maps <= 65535, DIHIP_PARAM_ERROR, "gqa_attn_mc: bad split / portion count");
  DIHIP_REQUIRE(!diff_out || (maps == 2 && ldd >= (long)H * DV && seq_dtype_ok(diff_dtype)), DIHIP_PARAM_ERROR,
                "gqa_attn_mc: the difference of the maps needs two maps and rows of H * DV elements");
  DIHIP_REQUIRE(ws_bytes >= dihip_gqa_attn_mc_workspace_bytes(T, H * maps, DV, nsplit) && (nsplit == 1 || ws), DIHIP_PARAM_ERROR,
                "gqa_attn_mc: workspace too small");
  if (E == 0 || max_count == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  GqaArgs a{out, ldo, q, ldq, kspans, vspans, span_stride, span_len, sink, w_dtype, sink_mode, softcap, gate, ldg, nullptr, tok_pos,
            ent_slot, ent_row0, ent_count, H, G, D, DV, scale, (float*)ws, T * H * maps, maps, window, keep_first};
  const int hpg = H / G, Dp = (D + 31) & ~31, Vp = (DV + 15) & ~15;
  const dim3 grid((unsigned)(((long)max_count * hpg + 63) / 64), E * G * maps, nsplit);
  const size_t lds = (size_t)32 * ((Dp + 8) + (Vp + 8)) * 2;
  auto go = [&](auto dm, auto vm) {
    constexpr int DM = decltype(dm)::value, VM = decltype(vm)::value;
    hipLaunchKernelGGL((gqa_attn_mc_kernel<DM, VM>), grid, dim3(256), lds, s, a);
  };
  auto by_v = [&](auto dm) {
    if (DV <= 64) go(dm, std::integral_constant<int, 64>{});
    else go(dm, std::integral_constant<int, 128>{});
  };
  if (D <= 64) by_v(std::integral_constant<int, 64>{});
  else if (D <= 128) by_v(std::integral_constant<int, 128>{});
  else by_v(std::integral_constant<int, 256>{});
  if (nsplit > 1 && diff_out)      // the merge of both maps, their difference and its norm in one launch
    hipLaunchKernelGGL(gqa_attn_merge_diff_kernel, dim3(T * H), dim3(256), 0, s, diff_out, diff_dtype, ldd, (const float*)ws, nsplit, T * H * maps, H, DV,
                       Vp, gate, ldg, lam, out_scale, eps);
  else if (nsplit > 1)
    hipLaunchKernelGGL(gqa_attn_merge_kernel, dim3(T * H * maps), dim3(256), 0, s, out, ldo, (const float*)ws, nsplit, T * H * maps, H, maps, DV, Vp, gate, ldg);
  else if (diff_out)
    hipLaunchKernelGGL(maps_diff_norm_kernel, dim3((unsigned)(((long)T * H + 3) / 4)), dim3(256), 0, s, diff_out, diff_dtype, ldd, out, ldo, lam, out_scale,
                       eps, T * H, H, DV);
  return launch_status();
}

int dihip_maps_diff_norm(void* stream, void* y, int y_dtype, long ldy, const float* x, long ldx, float lam, float out_scale, float eps, int T,
                         int H, int DV) {
  DIHIP_REQUIRE(T >= 0 && H > 0 && DV > 0 && y && x && ldy >= (long)H * DV && ldx >= (long)H * 2 * DV && seq_dtype_ok(y_dtype), DIHIP_PARAM_ERROR,
                "maps_diff_norm: bad argument");
  DIHIP_REQUIRE(DV <= 512, DIHIP_EXCEED_LIMIT_ERROR, "maps_diff_norm: heads of more than 512 values");
  if (T == 0) return DIHIP_SUCCESS;
  const long pairs = (long)T * H;
  hipLaunchKernelGGL(maps_diff_norm_kernel, dim3((unsigned)((pairs + 3) / 4)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), y, y_dtype, ldy,
                     x, ldx, lam, out_scale, eps, (int)pairs, H, DV);
  return launch_status();
}

}  // extern "C"
