// Attention over a cached LATENT: every token leaves one normed vector c (L elements) and one rotated key part
// kr (R elements) that all heads share; head a's key is [W_uk,a c | kr] and its value W_uv,a c. The products with
// W_uk and W_uv are moved to the query side and the output side:
//
//   score_a(i, j) = (W_uk,a^T q_plain,a(i)) . c_j + q_turned,a(i) . kr_j         out_a(i) = W_uv,a sum_j p_a(i, j) c_j
//
// so the attention itself runs over ONE key/value head whose key row is [c | kr] and whose value is c, and only
// c and kr are ever stored. Here: the kernel that finishes a token's projections (norm of c, rotation of kr and
// of the queries' rotated parts, cache write), and the per-head matrix product both sides use.
#include "tw_common.h"

// One rotated pair, products and sums spelled out (a*b - c*d left to the compiler becomes one fused form or the other).
__device__ __forceinline__ void lt_rotate_pair(float lo, float hi, float c, float s, float& out_lo, float& out_hi) {
  out_lo = __fmaf_rn(lo, c, -__fmul_rn(hi, s));
  out_hi = __fmaf_rn(hi, c, __fmul_rn(lo, s));
}

struct LatentFinishArgs {
  const void* proj; long ld;        // a token's projections: the heads' rotated query parts at q_col + a * Rp,
  int q_col, c_col, kr_col;         // the raw latent at c_col (L elements), the raw shared key part at kr_col
  const float* cos_t; const float* sin_t;    // [n][rot / 2]
  const float* norm_w;              // [L]
  void* q_out; long ld_q;           // [n][H][Lp + Rp]: this kernel fills columns Lp .. Lp + Rp of every head
  void* q_full; long ld_full;       // or null. [n][H][hd]: head a = [its D unrotated elements | its rotated part | zeros],
  int D, Dp, hd, full_from;         // for rows from full_from on (queries against keys expanded per head)
  void* keys; void* values;         // keys [pages][1][P][Lp + Rp], values [pages][1][Lp][P]; null: nothing is stored
  const int* slots;
  int H, L, Lp, Rp, rot, P;
  float eps;
};

template <typename T>
__global__ __launch_bounds__(256) void latent_finish_kernel(LatentFinishArgs a) {
  __shared__ float lds[16];
  const int n = blockIdx.x;
  const T* row = (const T*)a.proj + (size_t)n * a.ld;
  const int half = a.rot / 2;
  const float* cs = a.cos_t + (size_t)n * half;
  const float* sn = a.sin_t + (size_t)n * half;
  const int K = a.Lp + a.Rp;
  // the heads' rotated query parts
  T* q = (T*)a.q_out + (size_t)n * a.ld_q;
  for (int i = threadIdx.x; i < a.H * a.Rp; i += blockDim.x) {
    const int head = i / a.Rp, d = i % a.Rp;
    const T* src = row + a.q_col + head * a.Rp;
    float v;
    if (d < half) {
      float other;
      lt_rotate_pair(tw_to_float(src[d]), tw_to_float(src[d + half]), cs[d], sn[d], v, other);
    } else if (d < a.rot) {
      float other;
      lt_rotate_pair(tw_to_float(src[d - half]), tw_to_float(src[d]), cs[d - half], sn[d - half], other, v);
    } else {
      v = tw_to_float(src[d]);
    }
    q[(size_t)head * K + a.Lp + d] = tw_from_float<T>(v);
  }
  if (a.q_full && n >= a.full_from) {
    __syncthreads();                                                          // the rotated parts above, written by other threads
    T* qf = (T*)a.q_full + (size_t)n * a.ld_full;
    for (int i = threadIdx.x; i < a.H * a.hd; i += blockDim.x) {
      const int head = i / a.hd, d = i % a.hd;
      T v = tw_from_float<T>(0.f);
      if (d < a.D) v = row[head * a.Dp + d];                                   // (the unrotated parts lie first in the row)
      else if (d < a.D + a.rot) v = q[(size_t)head * K + a.Lp + d - a.D];
      qf[i] = v;
    }
  }
  if (!a.keys) return;
  const int slot = a.slots[n];
  // the latent's norm (every thread takes part in the sum, stored or not)
  float ss = 0.f;
  for (int i = threadIdx.x; i < a.L; i += blockDim.x) {
    const float v = tw_to_float(row[a.c_col + i]);
    ss = __fmaf_rn(v, v, ss);
  }
  const float total = tw_block_sum(ss, lds);
  if (slot < 0) return;
  const float rinv = 1.f / sqrtf(total / (float)a.L + a.eps);
  const int page = slot / a.P, at = slot % a.P;
  T* key = (T*)a.keys + ((size_t)page * a.P + at) * K;
  T* val = (T*)a.values + (size_t)page * a.Lp * a.P + at;
  for (int i = threadIdx.x; i < a.Lp; i += blockDim.x) {
    const T c = i < a.L ? tw_from_float<T>(tw_to_float(row[a.c_col + i]) * rinv * a.norm_w[i]) : tw_from_float<T>(0.f);
    key[i] = c;
    val[(size_t)i * a.P] = c;
  }
  for (int d = threadIdx.x; d < a.Rp; d += blockDim.x) {
    const T* src = row + a.kr_col;
    float v;
    if (d < half) {
      float other;
      lt_rotate_pair(tw_to_float(src[d]), tw_to_float(src[d + half]), cs[d], sn[d], v, other);
    } else if (d < a.rot) {
      float other;
      lt_rotate_pair(tw_to_float(src[d - half]), tw_to_float(src[d]), cs[d - half], sn[d - half], other, v);
    } else {
      v = 0.f;
    }
    key[a.Lp + d] = tw_from_float<T>(v);
  }
}

extern "C" int tw_latent_finish(int dtype, const void* proj, long ld, int q_col, int c_col, int kr_col,
                                const float* cos_t, const float* sin_t, const float* norm_w, void* q_out, long ld_q,
                                void* q_full, long ld_full, int D, int Dp, int hd, int full_from,
                                void* keys, void* values, const int* slots, int n, int H, int L, int Lp, int Rp, int rot,
                                int page_size, float eps, hipStream_t stream) {
  TW_REQUIRE(proj && cos_t && sin_t && q_out && n >= 0 && H > 0 && Rp > 0 && rot > 0 && rot % 2 == 0 && rot <= Rp);
  if (q_full) TW_REQUIRE(D > 0 && Dp >= D && hd >= D + rot && ld_full >= (long)H * hd && full_from >= 0 && q_col >= H * Dp);
  TW_REQUIRE(q_col >= 0 && ld >= q_col + (long)H * Rp && ld_q >= (long)H * (Lp + Rp) && Lp >= 0);
  if (keys) {
    TW_REQUIRE(values && slots && norm_w && L > 0 && Lp >= L && page_size > 0 && eps > 0.f);
    TW_REQUIRE(c_col >= 0 && kr_col >= 0 && ld >= c_col + (long)L && ld >= kr_col + (long)rot);
  }
  if (n == 0) return 0;
  LatentFinishArgs a{proj, ld, q_col, c_col, kr_col, cos_t, sin_t, norm_w, q_out, ld_q, q_full, ld_full, D, Dp, hd, full_from,
                     keys, values, slots, H, L, Lp, Rp, rot, page_size, eps};
  if (dtype == TW_DTYPE_BF16) latent_finish_kernel<bf16_t><<<n, 256, 0, stream>>>(a);
  else if (dtype == TW_DTYPE_F32) latent_finish_kernel<float><<<n, 256, 0, stream>>>(a);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- one small matrix per head: out[n][a * so + o] = sum_i x[n][a * sx + i] * w[a][o][i] ------------------------
// x and out hold the heads side by side, sx and so elements apart; w [heads][No][Ni] row-major. A wave takes 16
// rows and 64 output columns of one head; the weights are the A operand, so a lane ends with four consecutive
// output columns of one row. Sums are float32, rounded once to the compute type.
template <typename T>
__global__ __launch_bounds__(256) void head_linear_kernel(const T* __restrict__ x, long ldx, int sx, const T* __restrict__ w,
                                                          T* __restrict__ out, long ldo, int so, int n, int heads, int Ni,
                                                          int No, int col_groups) {
  typedef typename Elem<T>::Frag Frag;
  constexpr int EPF = Elem<T>::kPerFrag;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int unit = blockIdx.x * 4 + wave;
  const int head = unit / col_groups, cg = unit % col_groups;
  if (head >= heads) return;
  const int row = blockIdx.y * 16 + r;
  const int chunks = Ni / EPF, steps = (chunks + 3) / 4;
  const T* x_row = x + (size_t)(row < n ? row : 0) * ldx + (size_t)head * sx;
  f32x4 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int st = 0; st < steps; ++st) {
    const int chunk = st * 4 + g;
    const bool in = chunk < chunks;
    const Frag xf = (in && row < n) ? tw_load_frag(x_row + chunk * EPF) : Elem<T>::zero();
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int o = cg * 64 + t * 16 + r;
      const Frag wf = (in && o < No) ? tw_load_frag(w + ((size_t)head * No + o) * Ni + chunk * EPF) : Elem<T>::zero();
      tw_mma16(acc[t], wf, xf);                            // D[output 4g + e][row r]
    }
  }
  if (row >= n) return;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int o = cg * 64 + t * 16 + 4 * g;
    if (o < No) {
      T* dst = out + (size_t)row * ldo + (size_t)head * so + o;
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[e] = tw_from_float<T>(acc[t][e]);
    }
  }
}

extern "C" int tw_head_linear(int dtype, const void* x, long ldx, int sx, const void* w, void* out, long ldo, int so,
                              int n, int heads, int Ni, int No, hipStream_t stream) {
  const int epf = dtype == TW_DTYPE_BF16 ? 8 : 4;
  TW_REQUIRE(x && w && out && n >= 0 && heads > 0 && Ni > 0 && No > 0);
  TW_REQUIRE(dtype == TW_DTYPE_BF16 || dtype == TW_DTYPE_F32);
  TW_REQUIRE(Ni % epf == 0 && No % 4 == 0 && ldx % epf == 0 && sx % epf == 0 && sx >= 0 && so >= No);
  TW_REQUIRE(ldx >= (long)(heads - 1) * sx + Ni && ldo >= (long)(heads - 1) * so + No);
  TW_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0);
  if (n == 0) return 0;
  const int col_groups = tw_div_up(No, 64);
  const dim3 grid(tw_div_up((long)heads * col_groups, 4), tw_div_up(n, 16));
  if (dtype == TW_DTYPE_BF16)
    head_linear_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, sx, (const bf16_t*)w, (bf16_t*)out, ldo, so, n,
                                                         heads, Ni, No, col_groups);
  else
    head_linear_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, ldx, sx, (const float*)w, (float*)out, ldo, so, n,
                                                        heads, Ni, No, col_groups);
  return TW_LAUNCH_RESULT();
}

// ---- prompt portions: keys and values expanded per head for this step ------------------------------------------------
// Against many query rows it is cheaper to expand the cached latents once (k_a = W_uk,a c, v_a = W_uv,a c for every
// cached token of the sequences that bring a portion) and to run ordinary attention with one key/value head per
// query head than to carry the latent's size through every score. Two kernels around one matrix product:
//
//   latent_gather:        the key rows [c | kr] of sequences seq0 .. from their pages into rows of their own, sequence
//                         after sequence, each starting at a multiple of the page size (row = page of its own * P + place),
//                         and the block table of those pages
//   (product)             up[row] = [W_uk ; W_uv] c[row]
//   latent_expand_store:  keys [page][a][place][hd] = [up k-part of head a | kr | zeros], values [page][a][hd][place]
//                         = [up v-part | zeros]: the layout the attention kernels read
struct LatentGatherArgs {
  const void* keys;                  // [pages][1][P][K]
  const int* block_table; int table_stride;
  const int* kv_len; const int* kv_page_start;      // kv_page_start[s]: pages of their own before sequence s (all sequences of the step)
  void* rows;                        // [own pages * P][K]
  int* own_table; int own_stride;    // [>= seq0 + n_seqs][own_stride]
  int seq0, n_seqs, P, K;
};

template <typename T>
__global__ __launch_bounds__(256) void latent_gather_kernel(LatentGatherArgs a) {
  const int base = a.kv_page_start[a.seq0];
  const int pg = blockIdx.x;                                   // page of its own, counted from seq0's first
  int lo = a.seq0, hi = a.seq0 + a.n_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (a.kv_page_start[mid] - base <= pg) lo = mid; else hi = mid - 1;
  }
  const int s = lo, b = pg - (a.kv_page_start[s] - base);
  if (pg >= a.kv_page_start[a.seq0 + a.n_seqs] - base) return;
  if (threadIdx.x == 0) a.own_table[(size_t)s * a.own_stride + b] = pg;
  const int phys = a.block_table[(size_t)s * a.table_stride + b];
  const int live = min(a.P, a.kv_len[s] - b * a.P);
  const T* src = (const T*)a.keys + (size_t)(phys < 0 ? 0 : phys) * a.P * a.K;
  T* dst = (T*)a.rows + (size_t)pg * a.P * a.K;
  for (int i = threadIdx.x; i < a.P * a.K; i += blockDim.x)
    dst[i] = (phys >= 0 && i / a.K < live) ? src[i] : tw_from_float<T>(0.f);
}

extern "C" int tw_latent_gather(int dtype, const void* keys, const int* block_table, int table_stride, const int* kv_len,
                                const int* kv_page_start, void* rows, int* own_table, int own_stride, int seq0, int n_seqs,
                                int own_pages, int page_size, int K, hipStream_t stream) {
  TW_REQUIRE(keys && block_table && kv_len && kv_page_start && rows && own_table && seq0 >= 0 && n_seqs >= 0 && own_pages >= 0);
  TW_REQUIRE(page_size > 0 && K > 0 && own_stride > 0);
  if (n_seqs == 0 || own_pages == 0) return 0;
  LatentGatherArgs a{keys, block_table, table_stride, kv_len, kv_page_start, rows, own_table, own_stride, seq0, n_seqs, page_size, K};
  if (dtype == TW_DTYPE_BF16) latent_gather_kernel<bf16_t><<<own_pages, 256, 0, stream>>>(a);
  else if (dtype == TW_DTYPE_F32) latent_gather_kernel<float><<<own_pages, 256, 0, stream>>>(a);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// One workgroup a page: up [rows][H * D + H * E] (the heads' key parts, then their value parts), kr at rows[row][Lp ..].
template <typename T>
__global__ __launch_bounds__(256) void latent_expand_store_kernel(const T* __restrict__ up, long ld_up, const T* __restrict__ rows,
                                                                  int K, int Lp, T* __restrict__ keys, T* __restrict__ values,
                                                                  int H, int D, int R, int E, int hd, int P) {
  const int pg = blockIdx.x;
  T* kp = keys + (size_t)pg * H * P * hd;
  T* vp = values + (size_t)pg * H * hd * P;
  for (int i = threadIdx.x; i < H * P * hd; i += blockDim.x) {
    const int d = i % hd, t = (i / hd) % P, a = i / (hd * P);
    const size_t row = (size_t)pg * P + t;
    T v = tw_from_float<T>(0.f);
    if (d < D) v = up[row * ld_up + a * D + d];
    else if (d < D + R) v = rows[row * K + Lp + d - D];
    kp[i] = v;
  }
  for (int i = threadIdx.x; i < H * hd * P; i += blockDim.x) {
    const int t = i % P, e = (i / P) % hd, a = i / (P * hd);
    const size_t row = (size_t)pg * P + t;
    vp[i] = e < E ? up[row * ld_up + (size_t)H * D + a * E + e] : tw_from_float<T>(0.f);
  }
}

extern "C" int tw_latent_expand_store(int dtype, const void* up, long ld_up, const void* rows, int K, int Lp, void* keys,
                                      void* values, int own_pages, int H, int D, int R, int E, int hd, int page_size,
                                      hipStream_t stream) {
  TW_REQUIRE(up && rows && keys && values && own_pages >= 0 && H > 0 && D > 0 && R >= 0 && E > 0 && page_size > 0);
  TW_REQUIRE(hd >= D + R && hd >= E && ld_up >= (long)H * (D + E) && K >= Lp + R);
  if (own_pages == 0) return 0;
  if (dtype == TW_DTYPE_BF16)
    latent_expand_store_kernel<bf16_t><<<own_pages, 256, 0, stream>>>((const bf16_t*)up, ld_up, (const bf16_t*)rows, K, Lp,
                                                                      (bf16_t*)keys, (bf16_t*)values, H, D, R, E, hd, page_size);
  else if (dtype == TW_DTYPE_F32)
    latent_expand_store_kernel<float><<<own_pages, 256, 0, stream>>>((const float*)up, ld_up, (const float*)rows, K, Lp,
                                                                     (float*)keys, (float*)values, H, D, R, E, hd, page_size);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}
