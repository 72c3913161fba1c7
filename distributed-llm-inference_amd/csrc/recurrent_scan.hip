// Linear recurrences with a matrix state per head, S [key channel][value channel] in 32-bit,
// carried from token to token of a request in its state slot. Two rules, one kernel:
//
//   RULE_DELTA   u = k / sqrt(sum k^2 + 1e-6);  w = exp(-exp(-1/2) sigmoid(w_pre));  a = sigmoid(a_pre + a_bias)
//                S <- diag(w) S - (a * u) (u^T S) + k v^T   (both terms read the old S);   o = S^T r
//   RULE_BONUS   w = exp(-exp(w_pre));   o = (S + diag(bonus) k v^T)^T r;   S <- diag(w) S + k v^T
//
// followed, per token and head, by o / sqrt(mean(o^2) + eps) * norm_w * gate, with gate =
// sigmoid(g_pre) (RULE_DELTA) or silu(g_pre) (RULE_BONUS); the result is written in the type of
// the product that reads it. Everything here is 32-bit arithmetic on 32-bit inputs.
//
// One workgroup takes one (entry, head) and walks the entry's tokens in order. Thread
// (v, part) of D * PARTS threads keeps the D / PARTS state values S[part's keys][v] in registers:
// a column of S never leaves its PARTS neighbouring lanes, whose partial dot products meet in two
// lane swaps. The per-token vectors of up to TB tokens are staged in LDS at once (loads and
// transcendentals of a batch in parallel, the chain over tokens reads LDS only), and the batch's
// outputs are normalised and gated together afterwards. The sums of a token do not depend on
// where a step cut the request: the state is the only thing carried, and it is carried exactly.
//
// State slot layout: [heads][D (value)][D (key)] floats at `state + slot * state_stride`.
// A request whose first row of the step has position 0 starts from a zero state.
#include "common.h"

#define RULE_DELTA 0
#define RULE_BONUS 1

struct ScanArgs {
  const float* r; const float* k; const float* v;   // [rows][heads * D], each with its row stride
  const float* w_pre;                                // decay before its activation
  const float* a_pre; const float* a_bias;           // RULE_DELTA: removal rate before the sigmoid, its bias [heads * D]
  const float* g_pre;                                // gate before its activation
  int64_t r_stride, k_stride, v_stride, w_stride, a_stride, g_stride;
  const float* bonus;                                // RULE_BONUS: [heads][D]
  const float* norm_w;                               // [heads * D]
  float eps;
  float* state; int64_t state_stride;
  const int* q_start; const int* positions; const int* state_slots;
  void* out; int64_t out_stride;
  int heads;
};

template <typename T, int NK, int RULE>
__global__ __launch_bounds__(NK * 16) void recurrent_scan_kernel(ScanArgs p) {
  constexpr int PARTS = 4, D = NK * PARTS, TB = 8, THREADS = D * PARTS;
  __shared__ float sr[TB][D], sk[TB][D], sv[TB][D], sw[TB][D], sa[TB][D], so[TB][D];
  __shared__ float knorm[TB], onorm[TB];
  const int tid = threadIdx.x, vcol = tid / PARTS, part = tid % PARTS;
  const int lane = tid % DLI_WAVE, wave = tid / DLI_WAVE;
  constexpr int WAVES = THREADS / DLI_WAVE;  // whole waves: they make the sums over a head (THREADS >= 64)
  const int entry = blockIdx.x, head = blockIdx.y;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int64_t col0 = (int64_t)head * D;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * D + vcol) * D + part * NK;
  float s[NK];
  if (p.positions[row0] == 0) {
#pragma unroll
    for (int i = 0; i < NK; ++i) s[i] = 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < NK; ++i) s[i] = st[i];
  }

  for (int t0 = 0; t0 < n_rows; t0 += TB) {
    const int nb = min(TB, n_rows - t0);
    __syncthreads();  // the batch before is read out
    for (int idx = tid; idx < nb * D; idx += THREADS) {
      const int t = idx / D, c = idx - t * D;
      const int64_t row = row0 + t0 + t;
      sr[t][c] = p.r[row * p.r_stride + col0 + c];
      sk[t][c] = p.k[row * p.k_stride + col0 + c];
      sv[t][c] = p.v[row * p.v_stride + col0 + c];
      const float wp = p.w_pre[row * p.w_stride + col0 + c];
      if (RULE == RULE_DELTA) {
        sw[t][c] = expf(-0.6065306597126334f / (1.f + expf(-wp)));
        sa[t][c] = 1.f / (1.f + expf(-(p.a_pre[row * p.a_stride + col0 + c] + p.a_bias[col0 + c])));
      } else {
        sw[t][c] = expf(-expf(wp));
        sa[t][c] = p.bonus[col0 + c];
      }
    }
    __syncthreads();
    if (RULE == RULE_DELTA) {
      for (int t = wave; t < nb && wave < WAVES; t += WAVES) {
        float ss = 0.f;
        for (int c = lane; c < D; c += DLI_WAVE) ss += sk[t][c] * sk[t][c];
        ss = wave_sum(ss);
        if (lane == 0) knorm[t] = 1.f / sqrtf(ss + 1e-6f);
      }
      __syncthreads();
    }
    for (int t = 0; t < nb; ++t) {
      const float vv = sv[t][vcol];
      float o = 0.f;
      if (RULE == RULE_DELTA) {
        const float kn = knorm[t];
        float us = 0.f;
#pragma unroll
        for (int i = 0; i < NK; ++i) us = fmaf(sk[t][part * NK + i] * kn, s[i], us);
        us += __shfl_xor(us, 1, DLI_WAVE);
        us += __shfl_xor(us, 2, DLI_WAVE);
#pragma unroll
        for (int i = 0; i < NK; ++i) {
          const int c = part * NK + i;
          const float kk = sk[t][c], u = kk * kn;
          s[i] = sw[t][c] * s[i] - (sa[t][c] * u) * us + kk * vv;
          o = fmaf(s[i], sr[t][c], o);
        }
      } else {
#pragma unroll
        for (int i = 0; i < NK; ++i) {
          const int c = part * NK + i;
          const float kv = sk[t][c] * vv;
          o = fmaf(s[i] + sa[t][c] * kv, sr[t][c], o);
          s[i] = sw[t][c] * s[i] + kv;
        }
      }
      o += __shfl_xor(o, 1, DLI_WAVE);
      o += __shfl_xor(o, 2, DLI_WAVE);
      if (part == 0) so[t][vcol] = o;
    }
    __syncthreads();
    for (int t = wave; t < nb && wave < WAVES; t += WAVES) {
      float ss = 0.f;
      for (int c = lane; c < D; c += DLI_WAVE) ss += so[t][c] * so[t][c];
      ss = wave_sum(ss);
      if (lane == 0) onorm[t] = 1.f / sqrtf(ss / (float)D + p.eps);
    }
    __syncthreads();
    for (int idx = tid; idx < nb * D; idx += THREADS) {
      const int t = idx / D, c = idx - t * D;
      const int64_t row = row0 + t0 + t;
      const float g = p.g_pre[row * p.g_stride + col0 + c];
      const float gate = RULE == RULE_DELTA ? 1.f / (1.f + expf(-g)) : g / (1.f + expf(-g));
      ((T*)p.out)[row * p.out_stride + col0 + c] = from_f32<T>(so[t][c] * onorm[t] * p.norm_w[col0 + c] * gate);
    }
  }
#pragma unroll
  for (int i = 0; i < NK; ++i) st[i] = s[i];
}

template <typename T, int RULE>
static int launch_scan(const ScanArgs& p, int entries, int dim, hipStream_t stream) {
  const dim3 grid(entries, p.heads);
#define SCAN_CASE(NK) \
  case NK: recurrent_scan_kernel<T, NK, RULE><<<grid, NK * 16, 0, stream>>>(p); break;
  switch (dim / 4) {
    SCAN_CASE(4) SCAN_CASE(6) SCAN_CASE(8) SCAN_CASE(10) SCAN_CASE(12) SCAN_CASE(14) SCAN_CASE(16)
    SCAN_CASE(20) SCAN_CASE(24) SCAN_CASE(28) SCAN_CASE(32)
    default: return DLI_ERR_ARGUMENT;
  }
#undef SCAN_CASE
  return dli_launch_status();
}

// Head sizes that the kernel is built for.
extern "C" int dli_recurrent_scan_supports(int dim) {
  if (dim < 16 || dim % 8 != 0 || dim > 128) return 0;
  return dim <= 64 || dim % 16 == 0;
}

extern "C" int dli_recurrent_scan(const float* r, int64_t r_stride, const float* k, int64_t k_stride, const float* v,
                                  int64_t v_stride, const float* w_pre, int64_t w_stride, const float* a_pre,
                                  int64_t a_stride, const float* a_bias, const float* g_pre, int64_t g_stride,
                                  const float* bonus, const float* norm_w, float eps, float* state,
                                  int64_t state_stride, const int* q_start, const int* positions,
                                  const int* state_slots, void* out, int64_t out_stride, int entries, int heads,
                                  int dim, int rule, int out_is_bf16, hipStream_t stream) {
  if (entries <= 0) return DLI_OK;
  if (!dli_recurrent_scan_supports(dim) || heads <= 0 || heads > 65535 || (rule != RULE_DELTA && rule != RULE_BONUS) ||
      state_stride < (int64_t)heads * dim * dim || (rule == RULE_DELTA && (a_pre == nullptr || a_bias == nullptr)) ||
      (rule == RULE_BONUS && bonus == nullptr))
    return DLI_ERR_ARGUMENT;
  ScanArgs p;
  p.r = r; p.k = k; p.v = v; p.w_pre = w_pre; p.a_pre = a_pre; p.a_bias = a_bias; p.g_pre = g_pre;
  p.r_stride = r_stride; p.k_stride = k_stride; p.v_stride = v_stride; p.w_stride = w_stride;
  p.a_stride = a_stride; p.g_stride = g_stride;
  p.bonus = bonus; p.norm_w = norm_w; p.eps = eps; p.state = state; p.state_stride = state_stride;
  p.q_start = q_start; p.positions = positions; p.state_slots = state_slots; p.out = out; p.out_stride = out_stride;
  p.heads = heads;
  if (rule == RULE_DELTA)
    return out_is_bf16 ? launch_scan<bf16_t, RULE_DELTA>(p, entries, dim, stream)
                       : launch_scan<float, RULE_DELTA>(p, entries, dim, stream);
  return out_is_bf16 ? launch_scan<bf16_t, RULE_BONUS>(p, entries, dim, stream)
                     : launch_scan<float, RULE_BONUS>(p, entries, dim, stream);
}
