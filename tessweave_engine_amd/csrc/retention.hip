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
// kernel of one-token steps, where the step is bound by reading and writing S once (it walks longer rows too,
// slowly: the chunked kernel below is the one for prompt portions).
template <typename T, int NT>
__global__ __launch_bounds__(256) void retention_walk_kernel(RetentionArgs a, int seq0) {
  constexpr int DPW = 4 * NT;                       // key elements a wave
  __shared__ float raw[2][16 * NT];
  __shared__ float qk[2][16 * NT];
  __shared__ float red[4][64];
  const int slices = (a.Ep + 63) / 64;
  const int slice = blockIdx.x % slices;
  const int head = (blockIdx.x / slices) % a.H;
  const int s = seq0 + blockIdx.x / (slices * a.H);
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
static int retention_walk_launch(const RetentionArgs& a, int seq0, int n_seqs, hipStream_t stream) {
  const int slices = (a.Ep + 63) / 64;
  const dim3 grid((unsigned)n_seqs * a.H * slices);
  switch (a.Dp / 16) {
#define TW_RT_CASE(NT) case NT: retention_walk_kernel<T, NT><<<grid, 256, 0, stream>>>(a, seq0); break;
    TW_RT_CASE(1) TW_RT_CASE(2) TW_RT_CASE(3) TW_RT_CASE(4) TW_RT_CASE(5) TW_RT_CASE(6) TW_RT_CASE(7) TW_RT_CASE(8)
    TW_RT_CASE(9) TW_RT_CASE(10) TW_RT_CASE(11) TW_RT_CASE(12) TW_RT_CASE(13) TW_RT_CASE(14) TW_RT_CASE(15) TW_RT_CASE(16)
#undef TW_RT_CASE
    default: return TW_ERR_BAD_ARGUMENT;
  }
  return TW_LAUNCH_RESULT();
}

// Portions of prompts: a workgroup owns 64 value columns of one (sequence, head) and walks the portion in chunks of
// Bc tokens (64, or 32 for long keys). Per chunk, with i, j the tokens' places in it, n its tokens and g the decay:
//
//   P^T[j][i] = g^(i - j) k_j . q_i  (j <= i)            the waves share the 16 x 16 tiles out; through LDS to all
//   O^T[e][i] = sum_j V^T[e][j] P^T[j][i] + g^(i + 1) sum_d S[d][e] q_i[d]       wave w: columns 16 w .. of the slice
//   S[d][e]  <- g^n S[d][e] + sum_j g^(n - 1 - j) k_j[d] v_j[e]
//
// all on the matrix unit in float32 (16x16x4): P^T and S come out of one product in the register layout the
// next product wants as an operand, so nothing is transposed. S stays in registers from chunk to chunk (lane
// (g, r) of wave w holds S[16 t + 4 g + 0..3][16 w + r] for every tile t of the key elements).
template <typename T, int NT_MAX>
__global__ __launch_bounds__(256) void retention_chunk_kernel(RetentionArgs a, int seq0, int Bc) {
  extern __shared__ float rt_lds[];
  const int Dp = a.Dp, NT = Dp / 16;
  const int QS = Dp + 4, VS = 68, PS = Bc + 4;
  float* Qs = rt_lds;
  float* Ks = Qs + (size_t)Bc * QS;
  float* Vs = Ks + (size_t)Bc * QS;
  float* Ps = Vs + (size_t)Bc * VS;
  float* wgt = Ps + (size_t)Bc * PS;
  const int slices = (a.Ep + 63) / 64;
  const int slice = blockIdx.x % slices;
  const int head = (blockIdx.x / slices) % a.H;
  const int s = seq0 + blockIdx.x / (slices * a.H);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int first = a.q_start[s], last = a.q_start[s + 1];
  const float gamma = a.decay[head];
  const float lg = log2f(gamma);
  const int half = a.rot >> 1;
  const int e_col = slice * 64 + wave * 16 + r;              // this lane's value column as a B operand / S column
  const bool e_live = e_col < a.Ep;
  float* S_mem = a.state + ((size_t)a.state_slots[s] * a.H + head) * (size_t)Dp * a.Ep;
  f32x4 S[NT_MAX];
#pragma unroll
  for (int t = 0; t < NT_MAX; ++t) {
    S[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (t < NT && e_live) {
#pragma unroll
      for (int j = 0; j < 4; ++j) S[t][j] = S_mem[(size_t)(t * 16 + 4 * g + j) * a.Ep + e_col];
    }
  }
  for (int t0 = first; t0 < last; t0 += Bc) {
    const int nv = last - t0 < Bc ? last - t0 : Bc;          // tokens of this chunk
    const int nb = (nv + 15) / 16;                           // blocks of 16 tokens that hold any
    const int rows = nb * 16;
    // ---- this chunk's q and k (rotated, k scaled) and its values into LDS, rows past the end as zeros
    for (int idx = threadIdx.x; idx < rows * Dp; idx += 256) {
      const int i = idx / Dp, d = idx - i * Dp;
      float qv = 0.f, kv = 0.f;
      if (i < nv) {
        const T* row = (const T*)a.proj + (size_t)(t0 + i) * a.ld;
        const T* qp = row + a.q_col + head * Dp;
        const T* kp = row + a.k_col + head * Dp;
        qv = tw_to_float(qp[d]);
        kv = tw_to_float(kp[d]);
        if (d < a.rot) {
          const int pj = d < half ? d : d - half;
          const float c = a.cos_t[(size_t)(t0 + i) * half + pj], sn = a.sin_t[(size_t)(t0 + i) * half + pj];
          const int other = d < half ? d + half : d - half;
          const float qo = tw_to_float(qp[other]), ko = tw_to_float(kp[other]);
          if (d < half) {
            qv = __fmaf_rn(qv, c, -__fmul_rn(qo, sn));
            kv = __fmaf_rn(kv, c, -__fmul_rn(ko, sn));
          } else {
            qv = __fmaf_rn(qv, c, __fmul_rn(qo, sn));
            kv = __fmaf_rn(kv, c, __fmul_rn(ko, sn));
          }
        }
        kv *= a.k_scale;
      }
      Qs[i * QS + d] = qv;
      Ks[i * QS + d] = kv;
    }
    for (int idx = threadIdx.x; idx < rows * 64; idx += 256) {
      const int i = idx >> 6, e = idx & 63;
      float v = 0.f;
      if (i < nv && slice * 64 + e < a.Ep)
        v = tw_to_float(((const T*)a.proj)[(size_t)(t0 + i) * a.ld + a.v_col + head * a.Ep + slice * 64 + e]);
      Vs[i * VS + e] = v;
    }
    if (threadIdx.x < rows) wgt[threadIdx.x] = threadIdx.x < nv ? exp2f((float)(nv - 1 - (int)threadIdx.x) * lg) : 0.f;
    __syncthreads();
    // ---- P^T tiles (jb <= ib), shared out over the waves
    int tile = 0;
    for (int ib = 0; ib < nb; ++ib) {
      for (int jb = 0; jb <= ib; ++jb, ++tile) {
        if ((tile & 3) != wave) continue;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        const float* kr = Ks + (jb * 16 + r) * QS + 4 * g;
        const float* qr = Qs + (ib * 16 + r) * QS + 4 * g;
        for (int dk = 0; dk < NT; ++dk)
          tw_mma16(acc, *reinterpret_cast<const f32x4*>(kr + dk * 16), *reinterpret_cast<const f32x4*>(qr + dk * 16));
        const int i = ib * 16 + r;
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4) {
          const int j = jb * 16 + 4 * g + j4;
          Ps[j * PS + i] = j <= i ? acc[j4] * exp2f((float)(i - j) * lg) : 0.f;
        }
      }
    }
    __syncthreads();
    // ---- outputs of this chunk: O^T[e][i] for this wave's 16 columns
    for (int ib = 0; ib < nb; ++ib) {
      f32x4 intra = {0.f, 0.f, 0.f, 0.f}, cross = {0.f, 0.f, 0.f, 0.f};
      for (int jb = 0; jb <= ib; ++jb) {
        f32x4 va, pb;
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4) {
          va[j4] = Vs[(jb * 16 + 4 * g + j4) * VS + wave * 16 + r];
          pb[j4] = Ps[(jb * 16 + 4 * g + j4) * PS + ib * 16 + r];
        }
        tw_mma16(intra, va, pb);
      }
      const float* qr = Qs + (ib * 16 + r) * QS + 4 * g;
#pragma unroll
      for (int t = 0; t < NT_MAX; ++t)
        if (t < NT) tw_mma16(cross, S[t], *reinterpret_cast<const f32x4*>(qr + t * 16));
      const int i = ib * 16 + r;
      const int e0 = slice * 64 + wave * 16 + 4 * g;
      if (i < nv && e0 < a.Ep) {
        const float up = exp2f((float)(i + 1) * lg);
        f32x4 o;
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4) o[j4] = __fmaf_rn(up, cross[j4], intra[j4]);
        float* dst = a.out + (size_t)(t0 + i) * a.ld_out + head * a.Ep + e0;
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4)
          if (e0 + j4 < a.Ep) dst[j4] = o[j4];
      }
    }
    // ---- the state after this chunk
    const float all = exp2f((float)nv * lg);
#pragma unroll
    for (int t = 0; t < NT_MAX; ++t) {
      if (t < NT) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int jb = 0; jb < nb; ++jb) {
          f32x4 ka, vb;
#pragma unroll
          for (int j4 = 0; j4 < 4; ++j4) {
            const int j = jb * 16 + 4 * g + j4;
            ka[j4] = Ks[j * QS + t * 16 + r] * wgt[j];
            vb[j4] = Vs[j * VS + wave * 16 + r];
          }
          tw_mma16(acc, ka, vb);
        }
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4) S[t][j4] = __fmaf_rn(all, S[t][j4], acc[j4]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int t = 0; t < NT_MAX; ++t) {
    if (t < NT && e_live) {
#pragma unroll
      for (int j = 0; j < 4; ++j) S_mem[(size_t)(t * 16 + 4 * g + j) * a.Ep + e_col] = S[t][j];
    }
  }
}

static int retention_chunk_tokens(int Dp) { return Dp <= 128 ? 64 : 32; }

static size_t retention_chunk_lds(int Dp, int Bc) {
  return ((size_t)2 * Bc * (Dp + 4) + (size_t)Bc * 68 + (size_t)Bc * (Bc + 4) + Bc) * sizeof(float);
}

template <typename T, int NT_MAX>
static int retention_chunk_launch_nt(const RetentionArgs& a, int seq0, int n_seqs, hipStream_t stream) {
  const int Bc = retention_chunk_tokens(a.Dp);
  const size_t lds = retention_chunk_lds(a.Dp, Bc);
  static size_t allowed = 0;                       // per instantiation: the most dynamic LDS asked for so far
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)retention_chunk_kernel<T, NT_MAX>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    allowed = lds;
  }
  const int slices = (a.Ep + 63) / 64;
  retention_chunk_kernel<T, NT_MAX><<<dim3((unsigned)n_seqs * a.H * slices), 256, lds, stream>>>(a, seq0, Bc);
  return TW_LAUNCH_RESULT();
}

template <typename T>
static int retention_chunk_launch(const RetentionArgs& a, int seq0, int n_seqs, hipStream_t stream) {
  if (a.Dp <= 64) return retention_chunk_launch_nt<T, 4>(a, seq0, n_seqs, stream);
  if (a.Dp <= 128) return retention_chunk_launch_nt<T, 8>(a, seq0, n_seqs, stream);
  return retention_chunk_launch_nt<T, 16>(a, seq0, n_seqs, stream);
}

extern "C" int tw_retention(int dtype, const void* proj, long ld, int q_col, int k_col, int v_col, const float* cos_t,
                            const float* sin_t, int rot, const float* decay, float* state, const int* q_start,
                            const int* state_slots, float* out, long ld_out, int seq0, int n_seqs, int chunked, int H,
                            int Dp, int Ep, float k_scale, hipStream_t stream) {
  TW_REQUIRE(proj && decay && state && q_start && state_slots && out && n_seqs >= 0 && seq0 >= 0);
  TW_REQUIRE(H > 0 && Dp > 0 && Dp % 16 == 0 && Dp <= 256 && Ep > 0 && rot >= 0 && rot % 2 == 0 && rot <= Dp);
  TW_REQUIRE(rot == 0 || (cos_t && sin_t));
  TW_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && ld >= q_col + (long)H * Dp && ld >= k_col + (long)H * Dp &&
             ld >= v_col + (long)H * Ep && ld_out >= (long)H * Ep);
  if (n_seqs == 0) return 0;
  RetentionArgs a{proj, ld, q_col, k_col, v_col, cos_t, sin_t, rot, decay, state, q_start, state_slots, out, ld_out,
                  H, Dp, Ep, k_scale};
  if (chunked) {
    if (dtype == TW_DTYPE_BF16) return retention_chunk_launch<bf16_t>(a, seq0, n_seqs, stream);
    if (dtype == TW_DTYPE_F32) return retention_chunk_launch<float>(a, seq0, n_seqs, stream);
    return TW_ERR_BAD_ARGUMENT;
  }
  if (dtype == TW_DTYPE_BF16) return retention_walk_launch<bf16_t>(a, seq0, n_seqs, stream);
  if (dtype == TW_DTYPE_F32) return retention_walk_launch<float>(a, seq0, n_seqs, stream);
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
