// seq_gla.hip -- gated linear attention with a matrix state per head, everything in f32:
//   per head and row   alpha = sigmoid(z)^(1/tau)  (as exp(log sigmoid(z) / tau)),   S <- diag(alpha) S + k v^T,   o = S^T (q * q_scale)
// S [D, DV] lives per state slot and is carried from portion to portion.  The columns of S are independent, so a workgroup
// owns 64 columns of one head: thread (slice, column) keeps D / 4 rows of its column in registers; the decays, keys and
// queries of a row -- the same for every column -- are computed once into padded records and reach the state kernels through
// scalar loads; partial dot products of the four slices are summed in a fixed order.  Long portions are cut into chunks of
// 64 rows that run side by side: (1) every chunk composes its rows from S = 0 -> (product of its decays, the state it would end in), (2) the states the chunks really start from
// are carried over the chunks, (3) every chunk runs its rows from that state and writes the outputs.
// Beside it: the unit-RMS norm of every head's output times a multiplier (the output gate).
// The same state kernels serve a state-space mixer with one scalar decay per head (dihip_ssd): its rows kernel writes the records
//   decay = exp(-exp(a_log[h]) * dt) for every channel,  key = dt * B[group],  query = C[group],  dt = softplus(dt_raw + dt_bias[h]).
#include "seq_common.h"

namespace dihip {
namespace {

constexpr int GLA_CHUNK = 64, GLA_RB = 8;

struct GlaArgs {
  float* out; long ldo;
  const float* q; long ldq; const float* k; long ldk; const float* v; long ldv; const float* z; long ldz;
  float q_scale, inv_tau;
  float* state;                       // [slots][H][D][DV]
  const int32_t* ent_slot; const int32_t* ent_row0; const int32_t* ent_count;
  int H, D, DV, Dp, T;
  float* rec;                         // [T][H][3][Dp]: decay, key, scaled query of every row, padded with (1, 0, 0)
  float* ws; int max_chunks;          // ws: [E][max_chunks][H] records of D * DV (state) + D (decay product) floats
};

__device__ __forceinline__ float log_sigmoid(float z) { return -(log1pf(expf(-fabsf(z))) + fmaxf(-z, 0.f)); }

// What every column of a head needs of a row -- the decays, the keys and the scaled queries -- is the same for all lanes of
// a wave.  This kernel computes them once per row and channel into padded records; the state kernels then read them through
// uniform addresses (scalar loads into scalar registers: no LDS traffic and no vector instruction per operand).
__global__ __launch_bounds__(256) void gla_rows_kernel(GlaArgs a) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < a.H * a.Dp; c += 256) {
    const int h = c / a.Dp, i = c - h * a.Dp;
    float av = 1.f, kv = 0.f, qv = 0.f;
    if (i < a.D) {
      const size_t col = (size_t)h * a.D + i;
      av = expf(log_sigmoid(a.z[(size_t)t * a.ldz + col]) * a.inv_tau);
      kv = a.k[(size_t)t * a.ldk + col];
      qv = a.q[(size_t)t * a.ldq + col] * a.q_scale;
    }
    float* r = a.rec + ((size_t)t * a.H + h) * 3 * a.Dp + i;
    r[0] = av; r[a.Dp] = kv; r[2 * a.Dp] = qv;
  }
}

// The records of a state-space mixer: B and C [T, G * D] are shared by the heads of a group (head h reads group h / (H / G)).
__global__ __launch_bounds__(256) void ssd_rows_kernel(GlaArgs a, const float* __restrict__ dt, long lddt, const void* __restrict__ dt_bias,
                                                       const void* __restrict__ a_log, int wdt, int G) {
  const int t = blockIdx.x, hpg = a.H / G;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < a.H * a.Dp; c += 256 * gridDim.y) {     // few rows: a row's records spread over workgroups
    const int h = c / a.Dp, i = c - h * a.Dp;
    float av = 1.f, kv = 0.f, qv = 0.f;
    if (i < a.D) {
      const float x = dt[(size_t)t * lddt + h] + ld_any(dt_bias, h, wdt);
      const float step = x > 20.f ? x : log1pf(expf(x));
      const size_t col = (size_t)(h / hpg) * a.D + i;
      av = expf(-expf(ld_any(a_log, h, wdt)) * step);
      kv = step * a.k[(size_t)t * a.ldk + col];
      qv = a.q[(size_t)t * a.ldq + col];
    }
    float* r = a.rec + ((size_t)t * a.H + h) * 3 * a.Dp + i;
    r[0] = av; r[a.Dp] = kv; r[2 * a.Dp] = qv;
  }
}

typedef const __attribute__((address_space(4))) float* uniform_f32_ptr;   // read-only for the whole launch, uniform address: scalar loads

// PASS 0: the whole portion from the slot's state (writes outputs and the state).  PASS 1 / 3: see above.
// A workgroup of NS waves owns 64 * CPT columns of one head: thread (slice sl = wave, lane) keeps rows sl * DPT .. + DPT of the
// columns lane, lane + 64, ..: a row's operands are fetched once for CPT columns.
template <int DPT, int PASS, int CPT, int NS>
__global__ __launch_bounds__(64 * NS) void gla_kernel(GlaArgs a) {
  constexpr int CW = 64 * CPT, NT = 64 * NS;
  __shared__ float part[GLA_RB][NS][CW];
  const int tid = threadIdx.x, lane = tid & 63;
  const int sl = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int D = a.D, DV = a.DV, H = a.H, Dp = a.Dp;
  const int cbs = (DV + CW - 1) / CW;
  const int ch = blockIdx.x, h = blockIdx.y / cbs, cb = blockIdx.y - h * cbs, e = blockIdx.z;
  // the portion's bounds come through pointers of unknown address space: told to be wave-uniform, so that every address
  // derived from them is one too (else the records below would be fetched lane by lane)
  const int cnt = __builtin_amdgcn_readfirstlane(a.ent_count[e]), row0 = __builtin_amdgcn_readfirstlane(a.ent_row0[e]);
  const int lo = PASS == 0 ? 0 : ch * GLA_CHUNK;
  if (lo >= cnt) return;
  const int n = PASS == 0 ? cnt : min(GLA_CHUNK, cnt - lo);
  int j[CPT];
  bool col[CPT];
#pragma unroll
  for (int c = 0; c < CPT; ++c) { j[c] = cb * CW + c * 64 + lane; col[c] = j[c] < DV; }
  const bool slice_live = sl * DPT < D;     // (uniform) a slice of padding only has nothing to do
  const size_t recsz = (size_t)D * DV + D;
  float* wrec = PASS == 0 ? nullptr : a.ws + (((size_t)e * a.max_chunks + ch) * H + h) * recsz;
  float* sp = a.state + ((size_t)a.ent_slot[e] * H + h) * D * DV;
  float S[CPT][DPT], Ap[DPT];    // Ap (PASS 1): the product of the chunk's decays
#pragma unroll
  for (int ii = 0; ii < DPT; ++ii) Ap[ii] = 1.f;
#pragma unroll
  for (int c = 0; c < CPT; ++c)
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
      const int i = sl * DPT + ii;
      S[c][ii] = 0.f;
      if (PASS != 1 && col[c] && i < D) S[c][ii] = PASS == 0 ? sp[(size_t)i * DV + j[c]] : wrec[(size_t)i * DV + j[c]];
    }
  const float* vhead = a.v + (size_t)h * DV;
  for (int b0 = 0; b0 < n; b0 += GLA_RB) {
    const int nb = min(GLA_RB, n - b0);
    float vr[GLA_RB][CPT];
#pragma unroll
    for (int r = 0; r < GLA_RB; ++r)
#pragma unroll
      for (int c = 0; c < CPT; ++c) vr[r][c] = (r < nb && col[c]) ? vhead[(size_t)(row0 + lo + b0 + r) * a.ldv + j[c]] : 0.f;
    if (PASS != 1) __syncthreads();   // part of the batch before is no longer read
#pragma unroll
    for (int r = 0; r < GLA_RB; ++r) {
      if (r < nb) {
        float po[CPT];
#pragma unroll
        for (int c = 0; c < CPT; ++c) po[c] = 0.f;
        if (slice_live) {
          const uniform_f32_ptr rp = (uniform_f32_ptr)(a.rec + ((size_t)(row0 + lo + b0 + r) * H + h) * 3 * Dp + sl * DPT);
#pragma unroll
          for (int i0 = 0; i0 < DPT; i0 += 8) {
            float a8[8], k8[8], q8[8];
#pragma unroll
            for (int x = 0; x < 8; ++x) { a8[x] = rp[i0 + x]; k8[x] = rp[Dp + i0 + x]; }
            if (PASS != 1) {
#pragma unroll
              for (int x = 0; x < 8; ++x) q8[x] = rp[2 * Dp + i0 + x];
            }
#pragma unroll
            for (int x = 0; x < 8; ++x) {
              if (PASS == 1) Ap[i0 + x] *= a8[x];
#pragma unroll
              for (int c = 0; c < CPT; ++c) {
                S[c][i0 + x] = __builtin_fmaf(a8[x], S[c][i0 + x], k8[x] * vr[r][c]);
                if (PASS != 1) po[c] = __builtin_fmaf(S[c][i0 + x], q8[x], po[c]);
              }
            }
          }
        }
        if (PASS != 1) {
#pragma unroll
          for (int c = 0; c < CPT; ++c) part[r][sl][c * 64 + lane] = po[c];
        }
      }
    }
    if (PASS != 1) {
      __syncthreads();
      for (int u = tid; u < nb * CW; u += NT) {
        const int r = u / CW, c = u - r * CW;
        if (cb * CW + c < DV) {
          float sum;
          if constexpr (NS == 8) sum = ((part[r][0][c] + part[r][1][c]) + (part[r][2][c] + part[r][3][c])) + ((part[r][4][c] + part[r][5][c]) + (part[r][6][c] + part[r][7][c]));
          else sum = (part[r][0][c] + part[r][1][c]) + (part[r][2][c] + part[r][3][c]);
          a.out[(size_t)(row0 + lo + b0 + r) * a.ldo + (size_t)h * DV + cb * CW + c] = sum;
        }
      }
    }
  }
  if (PASS == 1 || PASS == 0 || lo + n == cnt) {
    float* dst = PASS == 1 ? wrec : sp;
#pragma unroll
    for (int c = 0; c < CPT; ++c)
#pragma unroll
      for (int ii = 0; ii < DPT; ++ii) {
        const int i = sl * DPT + ii;
        if (col[c] && i < D) dst[(size_t)i * DV + j[c]] = S[c][ii];
      }
  }
  if (PASS == 1 && cb == 0 && lane == 0) {
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
      const int i = sl * DPT + ii;
      if (i < D) wrec[(size_t)D * DV + i] = Ap[ii];
    }
  }
}

// pass 2: per state element, chunks in order: record <- the state the chunk starts from;  S <- decay product * S + record
__global__ __launch_bounds__(256) void gla_carry_kernel(GlaArgs a) {
  const int e = blockIdx.z, h = blockIdx.y;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.D * a.DV) return;
  const int i = idx / a.DV;
  const int chunks = (a.ent_count[e] + GLA_CHUNK - 1) / GLA_CHUNK;
  const size_t rec = (size_t)a.D * a.DV + a.D;
  float S = a.state[((size_t)a.ent_slot[e] * a.H + h) * a.D * a.DV + idx];
  const size_t step = (size_t)a.H * rec;
  float* w0 = a.ws + (((size_t)e * a.max_chunks) * a.H + h) * rec;
  constexpr int U8 = 8;     // eight chunks' records in flight: the chain itself is eight dependent multiply-adds
  for (int c0 = 0; c0 < chunks; c0 += U8) {
    float U[U8], A[U8];
#pragma unroll
    for (int x = 0; x < U8; ++x) {
      const int ch = min(c0 + x, chunks - 1);
      U[x] = w0[ch * step + idx];
      A[x] = w0[ch * step + (size_t)a.D * a.DV + i];
    }
#pragma unroll
    for (int x = 0; x < U8; ++x) {
      if (c0 + x < chunks) {
        w0[(c0 + x) * step + idx] = S;
        S = __builtin_fmaf(A[x], S, U[x]);
      }
    }
  }
}

template <int WT>
__global__ __launch_bounds__(256) void head_rmsnorm_mul_kernel(void* __restrict__ y, int ydt, long ldy, const float* __restrict__ x, long ldx,
                                                               const void* __restrict__ gamma, float eps, const float* __restrict__ mul,
                                                               long ldm, int H, int DV) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int h = blockIdx.y * 4 + wave; h < H; h += 4 * gridDim.y) {
    const float* xr = x + (size_t)t * ldx + (size_t)h * DV;
    float ss = 0.f;
    for (int d = lane; d < DV; d += 64) ss = __builtin_fmaf(xr[d], xr[d], ss);
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)DV + eps);
    for (int d = lane; d < DV; d += 64) {
      float v = xr[d] * inv * load_ft<WT>(gamma, d);
      if (mul) v *= mul[(size_t)t * ldm + (size_t)h * DV + d];
      st_any(y, (size_t)t * ldy + (size_t)h * DV + d, ydt, v);
    }
  }
}

}  // namespace
}  // namespace dihip

using namespace dihip;

extern "C" {

// columns per thread: two where the registers allow (D <= 128) and the head has more than 64 value columns -- and for 64 < D <= 128
// also where it has not: the one-column form of that size needs more registers than a lane has (it ran from scratch memory, ten
// times slower); the second column of such a thread is past the head and idle
static int gla_cpt(int D, int DV) { return D <= 128 && (DV > 64 || D > 64) ? 2 : 1; }
static int gla_dpad(int D) { return D <= 64 ? 64 : (D <= 128 ? 128 : 256); }

// the state kernels over records that a rows kernel has written
static void gla_launch_state(hipStream_t s, const GlaArgs& a, int E, int chunked, int cpt, int cbs) {
  const int H = a.H, D = a.D, DV = a.DV, chunks = a.max_chunks;
  const dim3 grid(chunks, H * cbs, E);
  // four slices of Dp / 4 channels; two columns per thread where the registers allow (D <= 128)
  auto go = [&](auto dpt, auto cp, auto ns) {
    constexpr int DPT = decltype(dpt)::value, CPT = decltype(cp)::value, NS = decltype(ns)::value;
    const dim3 block(64 * NS);
    if (!chunked) {
      hipLaunchKernelGGL((gla_kernel<DPT, 0, CPT, NS>), grid, block, 0, s, a);
    } else {
      hipLaunchKernelGGL((gla_kernel<DPT, 1, CPT, NS>), grid, block, 0, s, a);
      hipLaunchKernelGGL(gla_carry_kernel, dim3((D * DV + 255) / 256, H, E), dim3(256), 0, s, a);
      hipLaunchKernelGGL((gla_kernel<DPT, 3, CPT, NS>), grid, block, 0, s, a);
    }
  };
  using one = std::integral_constant<int, 1>;
  using two = std::integral_constant<int, 2>;
  using four = std::integral_constant<int, 4>;
  if (D <= 64) { if (cpt == 2) go(std::integral_constant<int, 16>{}, two{}, four{}); else go(std::integral_constant<int, 16>{}, one{}, four{}); }
  else if (D <= 128) { if (cpt == 2) go(std::integral_constant<int, 32>{}, two{}, four{}); else go(std::integral_constant<int, 32>{}, one{}, four{}); }
  else go(std::integral_constant<int, 64>{}, one{}, four{});
}

size_t dihip_gla_workspace_bytes(int T, int E, int max_count, int H, int D, int DV, int chunked) {
  size_t b = (size_t)T * H * 3 * gla_dpad(D) * sizeof(float);
  if (chunked) b += (size_t)E * ((max_count + GLA_CHUNK - 1) / GLA_CHUNK) * H * ((size_t)D * DV + D) * sizeof(float);
  return b;
}

int dihip_gla(void* stream, float* out, long ldo, const float* q, long ldq, const float* k, long ldk, const float* v, long ldv,
              const float* z, long ldz, float q_scale, float tau, float* state, const int32_t* ent_slot, const int32_t* ent_row0,
              const int32_t* ent_count, int T, int E, int max_count, int H, int D, int DV, int chunked, void* ws, size_t ws_bytes) {
  DIHIP_REQUIRE(T >= 0 && E >= 0 && max_count >= 0 && H > 0 && D > 0 && DV > 0 && out && q && k && v && z && state && ent_slot && ent_row0 &&
                    ent_count && ldo >= (long)H * DV && ldq >= (long)H * D && ldk >= (long)H * D && ldz >= (long)H * D && ldv >= (long)H * DV &&
                    tau > 0.f, DIHIP_PARAM_ERROR, "gla: bad argument");
  DIHIP_REQUIRE(D <= 256, DIHIP_EXCEED_LIMIT_ERROR, "gla: more than 256 key channels per head (%d)", D);
  const int cpt = gla_cpt(D, DV);
  const int cbs = (DV + 64 * cpt - 1) / (64 * cpt);
  DIHIP_REQUIRE((long)H * cbs <= 65535 && E <= 65535, DIHIP_PARAM_ERROR, "gla: too many heads or portions for one launch");
  DIHIP_REQUIRE(ws && ws_bytes >= dihip_gla_workspace_bytes(T, E, max_count, H, D, DV, chunked) && (reinterpret_cast<uintptr_t>(ws) & 3u) == 0,
                DIHIP_PARAM_ERROR, "gla: workspace too small");
  if (T == 0 || E == 0 || max_count == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int chunks = chunked ? (max_count + GLA_CHUNK - 1) / GLA_CHUNK : 1;
  const int Dp = gla_dpad(D);
  float* rec = (float*)ws;
  GlaArgs a{out, ldo, q, ldq, k, ldk, v, ldv, z, ldz, q_scale, 1.f / tau, state, ent_slot, ent_row0, ent_count, H, D, DV, Dp, T,
            rec, rec + (size_t)T * H * 3 * Dp, chunks};
  hipLaunchKernelGGL(gla_rows_kernel, dim3(T), dim3(256), 0, s, a);
  gla_launch_state(s, a, E, chunked, cpt, cbs);
  return launch_status();
}

int dihip_ssd(void* stream, float* out, long ldo, const float* x, long ldx, const float* B, long ldb, const float* Cq, long ldc, const float* dt,
              long lddt, const void* dt_bias, const void* a_log, int w_dtype, float* state, const int32_t* ent_slot, const int32_t* ent_row0,
              const int32_t* ent_count, int T, int E, int max_count, int H, int G, int D, int DV, int chunked, void* ws, size_t ws_bytes) {
  DIHIP_REQUIRE(T >= 0 && E >= 0 && max_count >= 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && DV > 0 && out && x && B && Cq && dt && dt_bias &&
                    a_log && state && ent_slot && ent_row0 && ent_count && ldo >= (long)H * DV && ldx >= (long)H * DV && ldb >= (long)G * D &&
                    ldc >= (long)G * D && lddt >= H && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "ssd: bad argument");
  DIHIP_REQUIRE(D <= 256, DIHIP_EXCEED_LIMIT_ERROR, "ssd: more than 256 state channels per head (%d)", D);
  const int cpt = gla_cpt(D, DV);
  const int cbs = (DV + 64 * cpt - 1) / (64 * cpt);
  DIHIP_REQUIRE((long)H * cbs <= 65535 && E <= 65535, DIHIP_PARAM_ERROR, "ssd: too many heads or portions for one launch");
  DIHIP_REQUIRE(ws && ws_bytes >= dihip_gla_workspace_bytes(T, E, max_count, H, D, DV, chunked) && (reinterpret_cast<uintptr_t>(ws) & 3u) == 0,
                DIHIP_PARAM_ERROR, "ssd: workspace too small");
  if (T == 0 || E == 0 || max_count == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int chunks = chunked ? (max_count + GLA_CHUNK - 1) / GLA_CHUNK : 1;
  const int Dp = gla_dpad(D);
  float* rec = (float*)ws;
  GlaArgs a{out, ldo, Cq, ldc, B, ldb, x, ldx, nullptr, 0, 1.f, 1.f, state, ent_slot, ent_row0, ent_count, H, D, DV, Dp, T,
            rec, rec + (size_t)T * H * 3 * Dp, chunks};
  hipLaunchKernelGGL(ssd_rows_kernel, dim3(T, T >= 64 ? 1 : (H * Dp + 255) / 256), dim3(256), 0, s, a, dt, lddt, dt_bias, a_log, w_dtype, G);
  gla_launch_state(s, a, E, chunked, cpt, cbs);
  return launch_status();
}

int dihip_head_rmsnorm_mul(void* stream, void* y, int y_dtype, long ldy, const float* x, long ldx, const void* gamma, int w_dtype,
                           float eps, const float* mul, long ldm, int T, int H, int DV) {
  DIHIP_REQUIRE(T >= 0 && H > 0 && DV > 0 && y && x && gamma && ldy >= (long)H * DV && ldx >= (long)H * DV && (!mul || ldm >= (long)H * DV) &&
                    seq_dtype_ok(y_dtype) && seq_dtype_ok(w_dtype), DIHIP_PARAM_ERROR, "head_rmsnorm_mul: bad argument");
  if (T == 0) return DIHIP_SUCCESS;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid(T, T >= 256 ? 1 : (H + 3) / 4);   // few rows (decoding): a wave per head; many rows: a workgroup per row
  if (w_dtype == DIHIP_F32) hipLaunchKernelGGL(head_rmsnorm_mul_kernel<DIHIP_F32>, grid, dim3(256), 0, s, y, y_dtype, ldy, x, ldx, gamma, eps, mul, ldm, H, DV);
  else hipLaunchKernelGGL(head_rmsnorm_mul_kernel<DIHIP_BF16>, grid, dim3(256), 0, s, y, y_dtype, ldy, x, ldx, gamma, eps, mul, ldm, H, DV);
  return launch_status();
}

}  // extern "C"
