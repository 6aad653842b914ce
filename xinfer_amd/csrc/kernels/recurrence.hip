// Linear attention with a decaying state (gated linear attention, retention): per request and head a
// matrix S [dk, dv] in float32 that every token updates and reads,
//
//     S <- diag(a_t) S + k_t v_t^T        o_t = S^T q_t
//
// with a_t a decay per key channel.  Two sources of the decay:
//   per head   a_t[i] = decay[h] for every token and channel (retention),
//   per token  a_t[i] = sigmoid(z_t[h, i])^(1 / tau) = exp(-softplus(-z) / tau), z float32 [T, H dk]
//              plus a bias [H dk] (gated linear attention); the logarithm, the exponential and the state
//              are float32.
// q, k and v are columns of a packed projection (a row stride and a column offset each); q and k are
// multiplied by `q_scale` / `k_scale` in float32 as they are read.
//
// `linear_scan_kernel`: one workgroup per (request, head, 64 value columns) walks the request's tokens of
// this step in order, from the state its slot holds, and leaves the new state there: the result does not
// depend on how a prompt was cut into steps or on what else is in the batch, bit for bit.  Lane l owns
// value column l of the tile, wave w the key channels w, w + 4, ..; a thread keeps its RPT state elements
// in registers for the whole walk.  A token costs one barrier: q, k and the decay of the next token are
// fetched while this one is worked on.
//
// `head_norm_gate_kernel`: what follows the state in both mixers: each head's o divided by its root mean
// square over dv (eps inside the root), times a weight [dv] shared by the heads (or none), times silu(g),
// rounded to the activation type for the output projection.
#include "common.h"

namespace xi {

constexpr int kScanWaves = 4;
constexpr int kScanCols = 64;

__device__ __forceinline__ float decay_of(float z, float inv_tau) {
  // sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau); softplus(x) = max(x, 0) + log1p(exp(-|x|))
  const float x = -z;
  const float sp = fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
  return expf(-sp * inv_tau);
}

template <typename T, int RPT>
__global__ __launch_bounds__(kScanWaves* kWave) void linear_scan_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ k, long long k_stride, const T* __restrict__ v,
    long long v_stride, const float* __restrict__ z, const float* __restrict__ z_bias, float inv_tau,
    const float* __restrict__ head_decay,
    float* __restrict__ state, long long slot_stride, const long long* __restrict__ state_slots,
    const int* __restrict__ cu_q, float* __restrict__ out, int H, int dk, int dv, float q_scale, float k_scale) {
  __shared__ float qs[2][kScanWaves * 64], ks[2][kScanWaves * 64], as[2][kScanWaves * 64];
  __shared__ float part[2][kScanWaves][kScanCols];
  const int b = blockIdx.x, h = blockIdx.y, j = blockIdx.z * kScanCols + (threadIdx.x & 63);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t0 = cu_q[b], t1 = cu_q[b + 1];
  if (t1 <= t0) return;
  const bool col = j < dv;
  float* S = state + (size_t)state_slots[b] * slot_stride + (size_t)h * dk * dv;
  float s[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int i = wave + kScanWaves * r;
    s[r] = (col && i < dk) ? S[(size_t)i * dv + j] : 0.f;
  }
  const int c = threadIdx.x;            // the channel this thread fetches for the workgroup
  const float hd = head_decay ? head_decay[h] : 0.f;
  const float zb = (z_bias && c < dk) ? z_bias[h * dk + c] : 0.f;
  auto fetch = [&](int t, float& fq, float& fk, float& fa) {
    if (c < dk) {
      fq = to_float(q[(size_t)t * q_stride + h * dk + c]) * q_scale;
      fk = to_float(k[(size_t)t * k_stride + h * dk + c]) * k_scale;
      fa = z ? decay_of(z[((size_t)t * H + h) * dk + c] + zb, inv_tau) : hd;
    }
  };
  float fq = 0.f, fk = 0.f, fa = 0.f;
  fetch(t0, fq, fk, fa);
  if (c < dk) {
    qs[0][c] = fq;
    ks[0][c] = fk;
    as[0][c] = fa;
  }
  __syncthreads();
  for (int t = t0; t < t1; ++t) {
    const int cur = (t - t0) & 1;
    if (t + 1 < t1) fetch(t + 1, fq, fk, fa);
    const float vj = col ? to_float(v[(size_t)t * v_stride + h * dv + j]) : 0.f;
    float acc = 0.f;
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
      const int i = wave + kScanWaves * r;
      if (i < dk) {
        s[r] = fmaf(as[cur][i], s[r], ks[cur][i] * vj);
        acc = fmaf(s[r], qs[cur][i], acc);
      }
    }
    part[cur][wave][lane] = acc;
    if (t + 1 < t1 && c < dk) {
      qs[cur ^ 1][c] = fq;
      ks[cur ^ 1][c] = fk;
      as[cur ^ 1][c] = fa;
    }
    __syncthreads();
    if (wave == 0 && col)
      out[((size_t)t * H + h) * dv + j] = (part[cur][0][lane] + part[cur][1][lane]) + (part[cur][2][lane] + part[cur][3][lane]);
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int i = wave + kScanWaves * r;
    if (col && i < dk) S[(size_t)i * dv + j] = s[r];
  }
}

// one wave per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             float eps, const T* __restrict__ g, long long g_stride,
                                                             T* __restrict__ out, long long pairs, int H, int dv) {
  const long long pair = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long long t = pair / H;
  const int h = (int)(pair - t * H);
  const float* x = o + (size_t)pair * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += kWave) ss = fmaf(x[i], x[i], ss);
  const float inv = rsqrtf(wave_sum(ss) / (float)dv + eps);
  const T* gr = g + (size_t)t * g_stride + (size_t)h * dv;
  T* orow = out + (size_t)pair * dv;
  for (int i = lane; i < dv; i += kWave) {
    const float gv = to_float(gr[i]);
    const float n = x[i] * inv * (w ? w[i] : 1.f);
    orow[i] = from_float<T>(n * (gv / (1.f + expf(-gv))));
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// q, k [T, .] with H dk columns from the given pointers, v with H dv, rows `*_stride` elements apart, in `dtype`;
// z float32 [T, H dk] (z_bias float32 [H dk] or null) or null (then head_decay float32 [H]); state float32, slot s at state + s * slot_stride,
// [H, dk, dv]; state_slots int64 [B]; cu_q int32 [B + 1]; out float32 [T, H, dv].
int xi_linear_scan(const void* q, long long q_stride, const void* k, long long k_stride, const void* v, long long v_stride,
                   int dtype, const float* z, const float* z_bias, float tau, const float* head_decay, float* state, long long slot_stride,
                   const long long* state_slots, const int* cu_q, float* out, int n_seqs, int H, int dk, int dv,
                   float q_scale, float k_scale, hipStream_t stream) {
  XI_CHECK(n_seqs >= 0 && H > 0 && dk > 0 && dv > 0, "linear_scan: bad sizes B=%d H=%d dk=%d dv=%d", n_seqs, H, dk, dv);
  XI_CHECK(dk <= kScanWaves * 64, "linear_scan: key heads of up to %d channels, not %d", kScanWaves * 64, dk);
  XI_CHECK((z != nullptr) != (head_decay != nullptr), "linear_scan: a decay per token or a decay per head, one of them");
  XI_CHECK(z == nullptr || tau > 0.f, "linear_scan: tau must be positive");
  XI_CHECK(slot_stride >= (long long)H * dk * dv, "linear_scan: a state slot is too small");
  if (n_seqs == 0) return 0;
  dim3 grid((unsigned)n_seqs, (unsigned)H, (unsigned)((dv + kScanCols - 1) / kScanCols));
  XI_CHECK(grid.y <= 65535u && grid.z <= 65535u, "linear_scan: too many heads or value columns");
  const float inv_tau = z ? 1.f / tau : 0.f;
  const int rpt = (dk + kScanWaves - 1) / kScanWaves;
#define XI_SCAN(TT, R)                                                                                                   \
  linear_scan_kernel<TT, R><<<grid, kScanWaves * kWave, 0, stream>>>(                                                    \
      (const TT*)q, q_stride, (const TT*)k, k_stride, (const TT*)v, v_stride, z, z_bias, inv_tau, head_decay, state, slot_stride, \
      state_slots, cu_q, out, H, dk, dv, q_scale, k_scale)
#define XI_SCAN_T(TT)            \
  do {                           \
    if (rpt <= 8) XI_SCAN(TT, 8); \
    else if (rpt <= 16) XI_SCAN(TT, 16); \
    else if (rpt <= 32) XI_SCAN(TT, 32); \
    else XI_SCAN(TT, 64);        \
  } while (0)
  if (dtype == kF32) XI_SCAN_T(float);
  else if (dtype == kBF16) XI_SCAN_T(bf16);
  else XI_CHECK(false, "linear_scan: unknown dtype %d", dtype);
#undef XI_SCAN_T
#undef XI_SCAN
  XI_LAUNCH_CHECK("linear_scan");
  return 0;
}

// o float32 [T, H, dv]; w float32 [dv] or null; g rows of g_stride elements holding [H dv] gates in `dtype`;
// out [T, H dv] in `dtype`.
int xi_head_norm_gate(const float* o, const float* w, float eps, const void* g, long long g_stride, void* out, int dtype,
                      int n_tok, int H, int dv, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0 && dv > 0 && g_stride >= (long long)H * dv, "head_norm_gate: bad sizes T=%d H=%d dv=%d", n_tok, H,
           dv);
  if (n_tok == 0) return 0;
  const long long pairs = (long long)n_tok * H;
  const long long blocks = (pairs + 3) / 4;
  XI_CHECK(blocks < (1ll << 31), "head_norm_gate: too many tokens");
  if (dtype == kF32)
    head_norm_gate_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(o, w, eps, (const float*)g, g_stride, (float*)out, pairs,
                                                                       H, dv);
  else if (dtype == kBF16)
    head_norm_gate_kernel<bf16><<<(unsigned)blocks, 256, 0, stream>>>(o, w, eps, (const bf16*)g, g_stride, (bf16*)out, pairs, H,
                                                                      dv);
  else
    XI_CHECK(false, "head_norm_gate: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

}  // extern "C"
