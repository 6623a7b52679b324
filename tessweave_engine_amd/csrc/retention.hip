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

// Portions of prompts: a workgroup owns 64 value columns of one (sequence, head, segment of the portion) and walks its
// segment in chunks of Bc tokens (32; 64 for keys of up to 64 elements: what keeps a workgroup's LDS under a third
// of a CU's). Per chunk, with i, j the tokens' places in it, n its tokens and g the decay:
//
//   P^T[j][i] = g^(i - j) k_j . q_i  (j <= i)            the waves share the 16 x 16 tiles out; through LDS to all
//   O^T[e][i] = sum_j V^T[e][j] P^T[j][i] + g^(i + 1) sum_d S[d][e] q_i[d]       wave w: columns 16 w .. of the slice
//   S[d][e]  <- g^n S[d][e] + sum_j g^(n - 1 - j) k_j[d] v_j[e]
//
// all on the matrix unit in float32 (16x16x4): P^T and S come out of one product in the register layout the
// next product wants as an operand, so nothing is transposed. S stays in registers from chunk to chunk (lane
// (g, r) of wave w holds S[16 t + 4 g + 0..3][16 w + r] for every tile t of the key elements).
//
// A long portion is cut into segments for separate workgroups, in two launches: LOCAL leaves, for every segment but
// a sequence's last, the state the segment alone would build from zero (the third line only); the main launch
// rebuilds each segment's true start from the request's state and the segments before it (in order), walks the
// segment, and the last segment writes the request's new state.
struct RetentionSegments {
  float* local;        // [sequence - seq0][H][segments][Dp][Ep]
  int seg_len;         // tokens a segment (a multiple of the chunk)
  int segments;        // the most segments a sequence of the launch has
};

// Rows of a chunk into LDS as float32: q and k rotated (k scaled), 8 elements a thread where everything is aligned.
template <typename T, bool WITH_Q>
__device__ __forceinline__ void rt_load_qk(const RetentionArgs& a, int head, int t0, int nv, int rows, float* Qs, float* Ks, int QS) {
  const int Dp = a.Dp, half = a.rot >> 1;
  const T* base = (const T*)a.proj;
  const bool vec = sizeof(T) == 2 && half % 8 == 0 && a.ld % 8 == 0 && a.q_col % 8 == 0 && a.k_col % 8 == 0 &&
                   ((uintptr_t)a.proj) % 16 == 0;
  if (vec) {
    const int groups = Dp / 8;
    for (int idx = threadIdx.x; idx < rows * groups; idx += 256) {
      const int i = idx / groups, d0 = (idx - i * groups) * 8;
      float qv[8], kv[8];
#pragma unroll
      for (int x = 0; x < 8; ++x) qv[x] = kv[x] = 0.f;
      if (i < nv) {
        const T* row = base + (size_t)(t0 + i) * a.ld + head * Dp;
        const bf16x8 kx = *reinterpret_cast<const bf16x8*>(row + a.k_col + d0);
        bf16x8 qx = kx;
        if (WITH_Q) qx = *reinterpret_cast<const bf16x8*>(row + a.q_col + d0);
        if (d0 < a.rot) {
          const int other = d0 < half ? d0 + half : d0 - half;
          const int pj = d0 < half ? d0 : d0 - half;
          const bf16x8 ko = *reinterpret_cast<const bf16x8*>(row + a.k_col + other);
          bf16x8 qo = ko;
          if (WITH_Q) qo = *reinterpret_cast<const bf16x8*>(row + a.q_col + other);
          const float* cs = a.cos_t + (size_t)(t0 + i) * half + pj;
          const float* sn = a.sin_t + (size_t)(t0 + i) * half + pj;
          const f32x4 c0 = *reinterpret_cast<const f32x4*>(cs), c1 = *reinterpret_cast<const f32x4*>(cs + 4);
          const f32x4 s0 = *reinterpret_cast<const f32x4*>(sn), s1 = *reinterpret_cast<const f32x4*>(sn + 4);
          const float sign = d0 < half ? -1.f : 1.f;
#pragma unroll
          for (int x = 0; x < 8; ++x) {
            const float c = x < 4 ? c0[x] : c1[x - 4], sv = sign * (x < 4 ? s0[x] : s1[x - 4]);
            kv[x] = __fmaf_rn((float)kx[x], c, __fmul_rn((float)ko[x], sv));
            if (WITH_Q) qv[x] = __fmaf_rn((float)qx[x], c, __fmul_rn((float)qo[x], sv));
          }
        } else {
#pragma unroll
          for (int x = 0; x < 8; ++x) {
            kv[x] = (float)kx[x];
            if (WITH_Q) qv[x] = (float)qx[x];
          }
        }
#pragma unroll
        for (int x = 0; x < 8; ++x) kv[x] *= a.k_scale;
      }
      float* kd = Ks + i * QS + d0;
      *reinterpret_cast<f32x4*>(kd) = f32x4{kv[0], kv[1], kv[2], kv[3]};
      *reinterpret_cast<f32x4*>(kd + 4) = f32x4{kv[4], kv[5], kv[6], kv[7]};
      if (WITH_Q) {
        float* qd = Qs + i * QS + d0;
        *reinterpret_cast<f32x4*>(qd) = f32x4{qv[0], qv[1], qv[2], qv[3]};
        *reinterpret_cast<f32x4*>(qd + 4) = f32x4{qv[4], qv[5], qv[6], qv[7]};
      }
    }
    return;
  }
  for (int idx = threadIdx.x; idx < rows * Dp; idx += 256) {
    const int i = idx / Dp, d = idx - i * Dp;
    float qv = 0.f, kv = 0.f;
    if (i < nv) {
      const T* row = base + (size_t)(t0 + i) * a.ld;
      const T* qp = row + a.q_col + head * Dp;
      const T* kp = row + a.k_col + head * Dp;
      qv = WITH_Q ? tw_to_float(qp[d]) : 0.f;
      kv = tw_to_float(kp[d]);
      if (d < a.rot) {
        const int pj = d < half ? d : d - half;
        const float c = a.cos_t[(size_t)(t0 + i) * half + pj], sn = a.sin_t[(size_t)(t0 + i) * half + pj];
        const int other = d < half ? d + half : d - half;
        const float qo = WITH_Q ? tw_to_float(qp[other]) : 0.f, ko = tw_to_float(kp[other]);
        const float sv = d < half ? -sn : sn;
        qv = __fmaf_rn(qv, c, __fmul_rn(qo, sv));
        kv = __fmaf_rn(kv, c, __fmul_rn(ko, sv));
      }
      kv *= a.k_scale;
    }
    if (WITH_Q) Qs[i * QS + d] = qv;
    Ks[i * QS + d] = kv;
  }
}

// NT_MAX: the most 16-element tiles of a key head this instance holds; EXACT: the head has exactly that many
// (loops over them have compile-time bounds and no conditions).
template <typename T, int NT_MAX, bool EXACT, bool LOCAL>
__global__ __launch_bounds__(256) void retention_chunk_kernel(RetentionArgs a, RetentionSegments sg, int seq0, int Bc) {
  extern __shared__ float rt_lds[];
  const int Dp = a.Dp;
  const int NT = EXACT ? NT_MAX : Dp / 16;
  const int QS = Dp + 4, VS = 68, PS = Bc + 4;
  float* Qs = rt_lds;
  float* Ks = Qs + (size_t)Bc * QS;
  float* Vs = Ks + (size_t)Bc * QS;
  float* Ps = Vs + (size_t)Bc * VS;
  float* wgt = Ps + (size_t)Bc * PS;
  const int slices = (a.Ep + 63) / 64;
  const int slice = blockIdx.x % slices;
  const int head = (blockIdx.x / slices) % a.H;
  const int s_local = blockIdx.x / (slices * a.H);
  const int s = seq0 + s_local;
  const int seg = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int q_first = a.q_start[s], q_last = a.q_start[s + 1];
  const int first = q_first + seg * sg.seg_len;
  if (first >= q_last) return;
  const bool final_seg = first + sg.seg_len >= q_last;
  if (LOCAL && final_seg) return;
  const int last = final_seg ? q_last : first + sg.seg_len;
  const float gamma = a.decay[head];
  const float lg = log2f(gamma);
  const int e_col = slice * 64 + wave * 16 + r;              // this lane's value column as a B operand / S column
  const bool e_live = e_col < a.Ep;
  float* S_mem = a.state + ((size_t)a.state_slots[s] * a.H + head) * (size_t)Dp * a.Ep;
  float* L_mem = sg.local + ((size_t)s_local * a.H + head) * (size_t)sg.segments * Dp * a.Ep;
  f32x4 S[NT_MAX];
#pragma unroll
  for (int t = 0; t < NT_MAX; ++t) {
    S[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (!LOCAL && t < NT && e_live) {
#pragma unroll
      for (int j = 0; j < 4; ++j) S[t][j] = S_mem[(size_t)(t * 16 + 4 * g + j) * a.Ep + e_col];
    }
  }
  if (!LOCAL && seg > 0) {
    // the segments before this one, in order: S <- g^seg_len S + what that segment alone built
    const float whole = exp2f((float)sg.seg_len * lg);
    for (int p = 0; p < seg; ++p) {
      const float* L = L_mem + (size_t)p * Dp * a.Ep;
#pragma unroll
      for (int t = 0; t < NT_MAX; ++t) {
        if (t < NT && e_live) {
#pragma unroll
          for (int j = 0; j < 4; ++j) S[t][j] = __fmaf_rn(whole, S[t][j], L[(size_t)(t * 16 + 4 * g + j) * a.Ep + e_col]);
        }
      }
    }
  }
  for (int t0 = first; t0 < last; t0 += Bc) {
    const int nv = last - t0 < Bc ? last - t0 : Bc;          // tokens of this chunk
    const int nb = (nv + 15) / 16;                           // blocks of 16 tokens that hold any
    const int rows = nb * 16;
    // ---- this chunk's q and k (rotated, k scaled) and its values into LDS, rows past the end as zeros
    rt_load_qk<T, !LOCAL>(a, head, t0, nv, rows, Qs, Ks, QS);
    for (int idx = threadIdx.x; idx < rows * 64; idx += 256) {
      const int i = idx >> 6, e = idx & 63;
      float v = 0.f;
      if (i < nv && slice * 64 + e < a.Ep)
        v = tw_to_float(((const T*)a.proj)[(size_t)(t0 + i) * a.ld + a.v_col + head * a.Ep + slice * 64 + e]);
      Vs[i * VS + e] = v;
    }
    if (threadIdx.x < rows) wgt[threadIdx.x] = threadIdx.x < nv ? exp2f((float)(nv - 1 - (int)threadIdx.x) * lg) : 0.f;
    __syncthreads();
    if (!LOCAL) {
      // ---- P^T tiles (jb <= ib), shared out over the waves
      int tile = 0;
      for (int ib = 0; ib < nb; ++ib) {
        for (int jb = 0; jb <= ib; ++jb, ++tile) {
          if ((tile & 3) != wave) continue;
          f32x4 acc = {0.f, 0.f, 0.f, 0.f};
          const float* kr = Ks + (jb * 16 + r) * QS + 4 * g;
          const float* qr = Qs + (ib * 16 + r) * QS + 4 * g;
#pragma unroll
          for (int dk = 0; dk < NT_MAX; ++dk)
            if (EXACT || dk < NT)
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
          if (EXACT || t < NT) tw_mma16(cross, S[t], *reinterpret_cast<const f32x4*>(qr + t * 16));
        const int i = ib * 16 + r;
        const int e0 = slice * 64 + wave * 16 + 4 * g;
        if (i < nv && e0 < a.Ep) {
          const float up = exp2f((float)(i + 1) * lg);
          float* dst = a.out + (size_t)(t0 + i) * a.ld_out + head * a.Ep + e0;
          if (e0 + 4 <= a.Ep) {
            f32x4 o;
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4) o[j4] = __fmaf_rn(up, cross[j4], intra[j4]);
            *reinterpret_cast<f32x4*>(dst) = o;
          } else {
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4)
              if (e0 + j4 < a.Ep) dst[j4] = __fmaf_rn(up, cross[j4], intra[j4]);
          }
        }
      }
    }
    // ---- the state after this chunk
    const float all = exp2f((float)nv * lg);
#pragma unroll
    for (int t = 0; t < NT_MAX; ++t) {
      if (EXACT || t < NT) {
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
  // With several segments the last one leaves the new state beside the others' (a workgroup of an earlier segment may
  // still have to read the old one); a small kernel moves it to the request's state afterwards.
  float* dst = (LOCAL || sg.segments > 1) ? L_mem + (size_t)seg * Dp * a.Ep : S_mem;
  if (LOCAL || final_seg) {
#pragma unroll
    for (int t = 0; t < NT_MAX; ++t) {
      if (t < NT && e_live) {
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[(size_t)(t * 16 + 4 * g + j) * a.Ep + e_col] = S[t][j];
      }
    }
  }
}

__global__ void retention_commit_kernel(RetentionArgs a, RetentionSegments sg, int seq0) {
  const int s_local = blockIdx.x / a.H, head = blockIdx.x % a.H;
  const int s = seq0 + s_local;
  const int q_len = a.q_start[s + 1] - a.q_start[s];
  if (q_len <= 0) return;
  const size_t count = (size_t)a.Dp * a.Ep;
  const float* src = sg.local + (((size_t)s_local * a.H + head) * sg.segments + (q_len - 1) / sg.seg_len) * count;
  float* dst = a.state + ((size_t)a.state_slots[s] * a.H + head) * count;
  for (size_t i = (size_t)blockIdx.y * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.y * blockDim.x) dst[i] = src[i];
}

static int retention_chunk_tokens(int Dp) { return Dp <= 64 ? 64 : 32; }

static size_t retention_chunk_lds(int Dp, int Bc) {
  return ((size_t)2 * Bc * (Dp + 4) + (size_t)Bc * 68 + (size_t)Bc * (Bc + 4) + Bc) * sizeof(float);
}

// Segments of a launch whose longest portion has max_q_len tokens: enough of them that the chip's CUs all have a
// workgroup, each at least four chunks long.
static void retention_segments(int n_seqs, int max_q_len, int H, int Dp, int Ep, int* seg_len, int* segments) {
  const int Bc = retention_chunk_tokens(Dp);
  const int chunks = tw_div_up(max_q_len, Bc);
  const long groups = (long)n_seqs * H * ((Ep + 63) / 64);
  long want = tw_div_up(1024, groups);
  if (want > chunks / 4) want = chunks / 4;
  if (want < 1) want = 1;
  const int per = tw_div_up(chunks, want);
  *seg_len = per * Bc;
  *segments = tw_div_up(chunks, per);
}

extern "C" long tw_retention_workspace_floats(int n_seqs, int max_q_len, int H, int Dp, int Ep) {
  if (n_seqs <= 0 || max_q_len <= 0) return 0;
  int seg_len, segments;
  retention_segments(n_seqs, max_q_len, H, Dp, Ep, &seg_len, &segments);
  return segments > 1 ? (long)n_seqs * H * segments * Dp * Ep : 0;
}

template <typename T, int NT_MAX, bool EXACT>
static int retention_chunk_launch_nt(const RetentionArgs& a, const RetentionSegments& sg, int seq0, int n_seqs, hipStream_t stream) {
  const int Bc = retention_chunk_tokens(a.Dp);
  const size_t lds = retention_chunk_lds(a.Dp, Bc);
  static size_t allowed = 0;                       // per instantiation: the most dynamic LDS asked for so far
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)retention_chunk_kernel<T, NT_MAX, EXACT, false>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)retention_chunk_kernel<T, NT_MAX, EXACT, true>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    allowed = lds;
  }
  const int slices = (a.Ep + 63) / 64;
  const dim3 grid((unsigned)n_seqs * a.H * slices, (unsigned)sg.segments);
  if (sg.segments > 1) retention_chunk_kernel<T, NT_MAX, EXACT, true><<<grid, 256, lds, stream>>>(a, sg, seq0, Bc);
  retention_chunk_kernel<T, NT_MAX, EXACT, false><<<grid, 256, lds, stream>>>(a, sg, seq0, Bc);
  if (sg.segments > 1) retention_commit_kernel<<<dim3((unsigned)n_seqs * a.H, 32), 256, 0, stream>>>(a, sg, seq0);
  return TW_LAUNCH_RESULT();
}

template <typename T>
static int retention_chunk_launch(const RetentionArgs& a, const RetentionSegments& sg, int seq0, int n_seqs, hipStream_t stream) {
  if (a.Dp == 64) return retention_chunk_launch_nt<T, 4, true>(a, sg, seq0, n_seqs, stream);
  if (a.Dp == 128) return retention_chunk_launch_nt<T, 8, true>(a, sg, seq0, n_seqs, stream);
  if (a.Dp == 256) return retention_chunk_launch_nt<T, 16, true>(a, sg, seq0, n_seqs, stream);
  if (a.Dp < 64) return retention_chunk_launch_nt<T, 4, false>(a, sg, seq0, n_seqs, stream);
  if (a.Dp < 128) return retention_chunk_launch_nt<T, 8, false>(a, sg, seq0, n_seqs, stream);
  return retention_chunk_launch_nt<T, 16, false>(a, sg, seq0, n_seqs, stream);
}

extern "C" int tw_retention(int dtype, const void* proj, long ld, int q_col, int k_col, int v_col, const float* cos_t,
                            const float* sin_t, int rot, const float* decay, float* state, const int* q_start,
                            const int* state_slots, float* out, long ld_out, int seq0, int n_seqs, int max_q_len, int H,
                            int Dp, int Ep, float k_scale, float* workspace, long workspace_floats, hipStream_t stream) {
  // max_q_len 0: the token-by-token kernel; else the chunked one, for portions of up to that many tokens
  TW_REQUIRE(proj && decay && state && q_start && state_slots && out && n_seqs >= 0 && seq0 >= 0 && max_q_len >= 0);
  TW_REQUIRE(H > 0 && Dp > 0 && Dp % 16 == 0 && Dp <= 256 && Ep > 0 && rot >= 0 && rot % 2 == 0 && rot <= Dp);
  TW_REQUIRE(rot == 0 || (cos_t && sin_t));
  TW_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && ld >= q_col + (long)H * Dp && ld >= k_col + (long)H * Dp &&
             ld >= v_col + (long)H * Ep && ld_out >= (long)H * Ep);
  if (n_seqs == 0) return 0;
  RetentionArgs a{proj, ld, q_col, k_col, v_col, cos_t, sin_t, rot, decay, state, q_start, state_slots, out, ld_out,
                  H, Dp, Ep, k_scale};
  if (max_q_len > 0) {
    TW_REQUIRE((uintptr_t)out % 16 == 0 && ld_out % 4 == 0);
    RetentionSegments sg{workspace, 0, 1};
    retention_segments(n_seqs, max_q_len, H, Dp, Ep, &sg.seg_len, &sg.segments);
    if (sg.segments > 1)
      TW_REQUIRE(workspace && workspace_floats >= tw_retention_workspace_floats(n_seqs, max_q_len, H, Dp, Ep));
    if (dtype == TW_DTYPE_BF16) return retention_chunk_launch<bf16_t>(a, sg, seq0, n_seqs, stream);
    if (dtype == TW_DTYPE_F32) return retention_chunk_launch<float>(a, sg, seq0, n_seqs, stream);
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
