// Retention: linear attention with a fixed decay per head, no softmax and no denominator.
//
//   S_t = decay_h * S_(t-1) + k_t v_t^T        (S: [D][E] per head and request, float32, carried from step to step)
//   o_t = S_t^T q_t
//
// q and k arrive unrotated in the compute type (a projection's result); they are rotated here in float32 with
// the step's cos/sin tables, k is then multiplied by k_scale, and from there everything is float32: the state,
// the decays, the products. A step's rows of one sequence are walked in order from the request's state, which
// the same workgroup reads at its start and writes at its end: nothing depends on how a prompt was cut.
//
// Heads are laid out with Dp = 16 * NT key elements and Ep value elements on the device (tails of zeros, which
// add nothing to a product and leave zero columns in S).
#include "tw_common.h"

struct RetentionArgs {
  const void* proj; long ld;          // a token's projections: q of head h at q_col + h * Dp, k at k_col + h * Dp,
  int q_col, k_col, v_col;            // v at v_col + h * Ep
  const float* cos_t; const float* sin_t; int rot;   // [n][rot / 2]; pair j is elements (j, j + rot / 2)
  const float* decay;                 // [H]
  float* state;                       // [requests][H][Dp][Ep]
  const int* q_start; const int* state_slots;
  float* out; long ld_out;            // float32 [n][>= H * Ep]: head h at h * Ep
  int H, Dp, Ep;
  float k_scale;
};

__device__ __forceinline__ float rt_rotated(const float* x, int d, int rot, const float* cs, const float* sn) {
  const int half = rot >> 1;
  if (d < half) return __fmaf_rn(x[d], cs[d], -__fmul_rn(x[d + half], sn[d]));
  if (d < rot) return __fmaf_rn(x[d], cs[d - half], __fmul_rn(x[d - half], sn[d - half]));
  return x[d];
}

// Token by token: a workgroup owns 64 value columns of one (sequence, head); lane = column, the four waves share
// the key elements out (wave w holds rows w * 4 NT .. of S in registers). Two barriers a token. This is the
// kernel of one-token steps, where the step is bound by reading and writing S once.
template <typename T, int NT>
__global__ __launch_bounds__(256) void retention_walk_kernel(RetentionArgs a) {
  constexpr int DPW = 4 * NT;                       // key elements a wave
  __shared__ float raw[2][16 * NT];
  __shared__ float qk[2][16 * NT];
  __shared__ float red[4][64];
  const int slices = (a.Ep + 63) / 64;
  const int slice = blockIdx.x % slices;
  const int head = (blockIdx.x / slices) % a.H;
  const int s = blockIdx.x / (slices * a.H);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e = slice * 64 + lane;
  const bool live = e < a.Ep;
  const int Dp = 16 * NT;
  const int first = a.q_start[s], last = a.q_start[s + 1];
  const float gamma = a.decay[head];
  float* S_mem = a.state + (((size_t)a.state_slots[s] * a.H + head) * Dp + wave * DPW) * a.Ep + e;
  float S[DPW];
#pragma unroll
  for (int i = 0; i < DPW; ++i) S[i] = live ? S_mem[(size_t)i * a.Ep] : 0.f;
  const int half = a.rot >> 1;
  for (int t = first; t < last; ++t) {
    const T* row = (const T*)a.proj + (size_t)t * a.ld;
    for (int i = threadIdx.x; i < 2 * Dp; i += blockDim.x) {
      const int which = i / Dp, d = i % Dp;
      raw[which][d] = tw_to_float(row[(which ? a.k_col : a.q_col) + head * Dp + d]);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * Dp; i += blockDim.x) {
      const int which = i / Dp, d = i % Dp;
      const float v = rt_rotated(raw[which], d, a.rot, a.cos_t + (size_t)t * half, a.sin_t + (size_t)t * half);
      qk[which][d] = which ? v * a.k_scale : v;
    }
    const float v_e = live ? tw_to_float(row[a.v_col + head * a.Ep + e]) : 0.f;
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < DPW; ++i) {
      const int d = wave * DPW + i;
      S[i] = __fmaf_rn(gamma, S[i], qk[1][d] * v_e);
      acc = __fmaf_rn(S[i], qk[0][d], acc);
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && live) a.out[(size_t)t * a.ld_out + head * a.Ep + e] = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DPW; ++i) S_mem[(size_t)i * a.Ep] = S[i];
  }
}

template <typename T>
static int retention_walk_launch(const RetentionArgs& a, int n_seqs, hipStream_t stream) {
  const int slices = (a.Ep + 63) / 64;
  const dim3 grid((unsigned)n_seqs * a.H * slices);
  switch (a.Dp / 16) {
#define TW_RT_CASE(NT) case NT: retention_walk_kernel<T, NT><<<grid, 256, 0, stream>>>(a); break;
    TW_RT_CASE(1) TW_RT_CASE(2) TW_RT_CASE(3) TW_RT_CASE(4) TW_RT_CASE(5) TW_RT_CASE(6) TW_RT_CASE(7) TW_RT_CASE(8)
    TW_RT_CASE(9) TW_RT_CASE(10) TW_RT_CASE(11) TW_RT_CASE(12) TW_RT_CASE(13) TW_RT_CASE(14) TW_RT_CASE(15) TW_RT_CASE(16)
#undef TW_RT_CASE
    default: return TW_ERR_BAD_ARGUMENT;
  }
  return TW_LAUNCH_RESULT();
}

extern "C" int tw_retention(int dtype, const void* proj, long ld, int q_col, int k_col, int v_col, const float* cos_t,
                            const float* sin_t, int rot, const float* decay, float* state, const int* q_start,
                            const int* state_slots, float* out, long ld_out, int n_seqs, int max_q_len, int H, int Dp,
                            int Ep, float k_scale, hipStream_t stream) {
  TW_REQUIRE(proj && decay && state && q_start && state_slots && out && n_seqs >= 0 && max_q_len >= 1);
  TW_REQUIRE(H > 0 && Dp > 0 && Dp % 16 == 0 && Dp <= 256 && Ep > 0 && rot >= 0 && rot % 2 == 0 && rot <= Dp);
  TW_REQUIRE(rot == 0 || (cos_t && sin_t));
  TW_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && ld >= q_col + (long)H * Dp && ld >= k_col + (long)H * Dp &&
             ld >= v_col + (long)H * Ep && ld_out >= (long)H * Ep);
  if (n_seqs == 0) return 0;
  RetentionArgs a{proj, ld, q_col, k_col, v_col, cos_t, sin_t, rot, decay, state, q_start, state_slots, out, ld_out,
                  H, Dp, Ep, k_scale};
  if (dtype == TW_DTYPE_BF16) return retention_walk_launch<bf16_t>(a, n_seqs, stream);
  if (dtype == TW_DTYPE_F32) return retention_walk_launch<float>(a, n_seqs, stream);
  return TW_ERR_BAD_ARGUMENT;
}

// ---- each head's result over its root mean square, times silu of a gate ------------------------------------------
// out[n][h * Ep + e] = o[n][h * Ep + e] / sqrt(mean_e(o^2) + eps) * silu(gate[n][h * Ep + e]); the mean runs over
// the head's E real elements (the device layout's tail is zeros and stays zeros). One wave a (token, head).
template <typename T>
__global__ __launch_bounds__(256) void unit_gate_kernel(const float* __restrict__ o, long ld_o, const T* __restrict__ gate,
                                                        long ld_g, T* __restrict__ out, long ld_out, int n, int H, int E,
                                                        int Ep, float eps) {
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= n * H) return;
  const int lane = threadIdx.x & 63;
  const int row = unit / H, head = unit % H;
  const float* src = o + (size_t)row * ld_o + (size_t)head * Ep;
  float ss = 0.f;
  for (int e = lane; e < E; e += 64) ss = __fmaf_rn(src[e], src[e], ss);
  ss = tw_wave_sum(ss);
  const float rinv = 1.f / sqrtf(ss / (float)E + eps);
  const T* g = gate + (size_t)row * ld_g + (size_t)head * Ep;
  T* dst = out + (size_t)row * ld_out + (size_t)head * Ep;
  for (int e = lane; e < Ep; e += 64) {
    float v = 0.f;
    if (e < E) {
      const float z = tw_to_float(g[e]);
      v = src[e] * rinv * (z / (1.f + expf(-z)));
    }
    dst[e] = tw_from_float<T>(v);
  }
}

extern "C" int tw_unit_gate(int dtype, const float* o, long ld_o, const void* gate, long ld_g, void* out, long ld_out,
                            int n, int H, int E, int Ep, float eps, hipStream_t stream) {
  TW_REQUIRE(o && gate && out && n >= 0 && H > 0 && E > 0 && Ep >= E && eps > 0.f);
  TW_REQUIRE(ld_o >= (long)H * Ep && ld_g >= (long)H * Ep && ld_out >= (long)H * Ep);
  if (n == 0) return 0;
  const int blocks = tw_div_up((long)n * H, 4);
  if (dtype == TW_DTYPE_BF16)
    unit_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(o, ld_o, (const bf16_t*)gate, ld_g, (bf16_t*)out, ld_out, n, H, E, Ep, eps);
  else if (dtype == TW_DTYPE_F32)
    unit_gate_kernel<float><<<blocks, 256, 0, stream>>>(o, ld_o, (const float*)gate, ld_g, (float*)out, ld_out, n, H, E, Ep, eps);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}
