// The gated delta rule: a recurrent mixer whose state is a matrix S [key channels, value channels] per head.
//
//   S <- g * S           g: one decay per head, or one per head and key channel (it scales rows of S)
//   u  = beta (v - S^T k)
//   S <- S + k u^T
//   o  = S^T q           the read-out sees the token's own write
//
// Three kernels run a step of any number of tokens per sequence, all in float32:
//   delta_prepare:  the short causal convolution over time of the q, k and v channels (inputs before the step come
//                   from the sequence's state, zeros before its start), silu, unit vectors per q and k head, q's scale,
//                   beta = sigmoid, g = exp(-exp(A_log) softplus(a + dt_bias)).
//   conv_state:     the last (taps - 1) inputs of every sequence go into its state.
//   delta_rule:     the recurrence.  Columns of S never mix (each value channel is a recurrence of its own), so a wave
//                   owns a few columns of one head of one sequence: 16 lanes share a column, each with a run of its
//                   rows in registers.  The wave walks over the sequence's tokens; q, k and g of a run of tokens are
//                   staged in LDS for all its lanes.  With kg = g k and qg = g q, both inner products of a token read
//                   the state as the token found it,  u = beta (v - S^T kg),  o = S^T qg + (k . q) u,  and are summed
//                   over the 16 lanes together; then S <- g S + k u^T.
//   gated_head_norm: o / rms(o) * weight * act(gate) per head, rounded once to the activation type.
//
// The state is kept transposed, [slot][head][value channel][key channel], so that a lane's rows are contiguous.
#include "common.h"
#include "fmsamd.h"

#define DELTA_MAX_TAPS 8

__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float sigmoid_f32(float z) { return 1.f / (1.f + expf(-z)); }

template <typename W>
__global__ void __launch_bounds__(256)
    delta_prepare_kernel(const float* __restrict__ proj, long ld, int col_b, const float* __restrict__ a, long lda, int col_a,
                         const W* __restrict__ conv_w, int taps, const float* __restrict__ a_log,
                         const float* __restrict__ dt_bias, const float* __restrict__ conv_state,
                         const int* __restrict__ seq_of_token, const int* __restrict__ slot_ids, float* __restrict__ qkv,
                         float* __restrict__ beta, float* __restrict__ decay, int H, int G, int D, int Dv, int per_channel,
                         float q_scale) {
  extern __shared__ float y[];  // the C convolved channels of this token
  const int t = blockIdx.x;
  const int seq = seq_of_token[t];
  if (seq < 0) return;
  const int slot = slot_ids[seq];
  const int C = 2 * G * D + H * Dv;
  // how many tokens of this sequence come before this one in the step (all that matters: up to taps - 1)
  int have = 0;
  for (int d = 1; d < taps; ++d) {
    if (t - d >= 0 && seq_of_token[t - d] == seq) have = d;
    else break;
  }
  const float* state = conv_state + (size_t)slot * (taps - 1) * C;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int d = taps - 1 - j;  // how far back this tap reaches
      const float x = d <= have ? proj[(size_t)(t - d) * ld + c] : state[(size_t)(taps - 1 + have - d) * C + c];
      acc = fmaf(to_f32(conv_w[(size_t)c * taps + j]), x, acc);
    }
    y[c] = acc / (1.f + expf(-acc));
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  for (int head = wave; head < 2 * G; head += nwaves) {
    float* v = y + (size_t)head * D;
    float s = 0.f;
    for (int i = lane; i < D; i += WAVE) s = fmaf(v[i], v[i], s);
    s = wave_sum(s);
    const float inv = (head < G ? q_scale : 1.f) / sqrtf(s + 1e-6f);
    for (int i = lane; i < D; i += WAVE) v[i] *= inv;
  }
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += blockDim.x) qkv[(size_t)t * C + c] = y[c];
  for (int h = threadIdx.x; h < H; h += blockDim.x) beta[(size_t)t * H + h] = sigmoid_f32(proj[(size_t)t * ld + col_b + h]);
  const int per_head = per_channel ? D : 1;
  for (int i = threadIdx.x; i < H * per_head; i += blockDim.x) {
    const float z = a[(size_t)t * lda + col_a + i] + dt_bias[i];
    decay[(size_t)t * H * per_head + i] = expf(-expf(a_log[i / per_head]) * softplus_f32(z));
  }
}

// Runs after delta_prepare of the same step (which reads the old state).  The block of a sequence's last token of the
// step writes; new entry s reads either a row of the step or an old entry above s, so ascending order is safe in place.
__global__ void __launch_bounds__(256)
    conv_state_kernel(const float* __restrict__ proj, long ld, int taps, float* __restrict__ conv_state,
                      const int* __restrict__ seq_of_token, const int* __restrict__ slot_ids, int n_tokens, int C) {
  const int t = blockIdx.x;
  const int seq = seq_of_token[t];
  if (seq < 0) return;
  if (t + 1 < n_tokens && seq_of_token[t + 1] == seq) return;  // not the sequence's last token of the step
  int have = 0;
  for (int d = 1; d < taps; ++d) {
    if (t - d >= 0 && seq_of_token[t - d] == seq) have = d;
    else break;
  }
  float* state = conv_state + (size_t)slot_ids[seq] * (taps - 1) * C;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    for (int s = 0; s < taps - 1; ++s) {
      const int d = taps - 2 - s;  // new entry s is the input d tokens before the last one
      state[(size_t)s * C + c] = d <= have ? proj[(size_t)(t - d) * ld + c] : state[(size_t)(taps - 1 + have - d) * C + c];
    }
  }
}

// --------------------------------------------------------------------------
// the recurrence
// --------------------------------------------------------------------------
#define DELTA_PARTS 16                      // lanes that share a column of S
#define DELTA_COLS (WAVE / DELTA_PARTS)     // columns of S a wave owns

struct DeltaArgs {
  const float* qkv;    // [T, C]: q [G*D] | k [G*D] | v [H*Dv]
  const float* beta;   // [T, H]
  const float* decay;  // [T, H] or [T, H*D]
  float* state;        // [slots][H][Dv][D]
  float* out;          // [T, H*Dv]
  const int* seq_starts;
  const int* seq_of_token;
  const int* slot_ids;
  int H, G, D, Dv, per_channel;
};

// R: rows of S per lane (D <= 16 R).  TC: tokens staged at a time.
template <int R, int TC>
__global__ void __launch_bounds__(WAVE) delta_rule_kernel(DeltaArgs a) {
  constexpr int DP = R * DELTA_PARTS;  // padded key size
  __shared__ __attribute__((aligned(16))) float qg[TC][DP];
  __shared__ __attribute__((aligned(16))) float kg[TC][DP];
  __shared__ __attribute__((aligned(16))) float kk[TC][DP];
  __shared__ __attribute__((aligned(16))) float gg[TC][DP];
  __shared__ float vv[TC][DELTA_COLS];
  __shared__ float bb[TC];
  __shared__ float kq[TC];
  __shared__ float oo[TC][DELTA_COLS];

  const int b = blockIdx.x, h = blockIdx.y;
  const int t0 = a.seq_starts[b], t1 = a.seq_starts[b + 1];
  if (t0 >= t1 || a.seq_of_token[t0] < 0) return;
  const int slot = a.slot_ids[b];
  const int lane = threadIdx.x;
  const int part = lane % DELTA_PARTS, col = lane / DELTA_PARTS;
  const int j = blockIdx.z * DELTA_COLS + col;  // this lane's column of S
  const int H = a.H, G = a.G, D = a.D, Dv = a.Dv;
  const int C = 2 * G * D + H * Dv;
  const int kh = h / (H / G);
  const bool live = j < Dv;

  float S[R];
  float* srow = a.state + (((size_t)slot * H + h) * Dv + (live ? j : 0)) * D + part * R;
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = (live && part * R + r < D) ? srow[r] : 0.f;

  for (int tb = t0; tb < t1; tb += TC) {
    const int n = t1 - tb < TC ? t1 - tb : TC;
    __syncthreads();  // the last run's reads are done
    for (int idx = lane; idx < n * DP; idx += WAVE) {
      const int tt = idx / DP, i = idx % DP;
      float q = 0.f, k = 0.f, g = 0.f;
      if (i < D) {
        const float* row = a.qkv + (size_t)(tb + tt) * C;
        q = row[kh * D + i];
        k = row[G * D + kh * D + i];
        g = a.per_channel ? a.decay[((size_t)(tb + tt) * H + h) * D + i] : a.decay[(size_t)(tb + tt) * H + h];
      }
      qg[tt][i] = q * g;
      kg[tt][i] = k * g;
      kk[tt][i] = k;
      gg[tt][i] = g;
    }
    for (int idx = lane; idx < n * DELTA_COLS; idx += WAVE) {
      const int tt = idx / DELTA_COLS, c = idx % DELTA_COLS;
      const int jj = blockIdx.z * DELTA_COLS + c;
      vv[tt][c] = jj < Dv ? a.qkv[(size_t)(tb + tt) * C + 2 * G * D + h * Dv + jj] : 0.f;
    }
    if (lane < n) bb[lane] = a.beta[(size_t)(tb + lane) * H + h];
    // k . q of every staged token: TC tokens x 64 / TC lanes each
    {
      constexpr int LPT = WAVE / TC;  // lanes per token
      const int tt = lane / LPT, sub = lane % LPT;
      float s = 0.f;
      if (tt < n) {
        const float* row = a.qkv + (size_t)(tb + tt) * C;
        for (int i = sub; i < D; i += LPT) s = fmaf(row[kh * D + i], row[G * D + kh * D + i], s);
      }
#pragma unroll
      for (int off = LPT / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, WAVE);
      if (sub == 0) kq[tt] = s;
    }
    __syncthreads();

    for (int tt = 0; tt < n; ++tt) {
      float du = 0.f, dq = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        du = fmaf(S[r], kg[tt][part * R + r], du);
        dq = fmaf(S[r], qg[tt][part * R + r], dq);
      }
#pragma unroll
      for (int off = DELTA_PARTS / 2; off > 0; off >>= 1) {
        du += __shfl_xor(du, off, WAVE);
        dq += __shfl_xor(dq, off, WAVE);
      }
      const float u = bb[tt] * (vv[tt][col] - du);
#pragma unroll
      for (int r = 0; r < R; ++r) S[r] = fmaf(kk[tt][part * R + r], u, gg[tt][part * R + r] * S[r]);
      if (part == 0) oo[tt][col] = fmaf(kq[tt], u, dq);
    }
    __syncthreads();
    for (int idx = lane; idx < n * DELTA_COLS; idx += WAVE) {
      const int tt = idx / DELTA_COLS, c = idx % DELTA_COLS;
      const int jj = blockIdx.z * DELTA_COLS + c;
      if (jj < Dv) a.out[(size_t)(tb + tt) * H * Dv + h * Dv + jj] = oo[tt][c];
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (part * R + r < D) srow[r] = S[r];
  }
}

// out[t, h, j] = o / rms_j(o) * weight[j] * act(gate[t, h, j]) * out_scale; one wave per (token, head)
template <typename T, typename W>
__global__ void __launch_bounds__(256)
    gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate, long ldg, const W* __restrict__ weight,
                           float eps, int act, float out_scale, T* __restrict__ out, long ldo, const int* __restrict__ seq_of_token,
                           int n_tokens, int H, int Dv) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long pair = (long)blockIdx.x * 4 + wave;
  if (pair >= (long)n_tokens * H) return;
  const int t = (int)(pair / H), h = (int)(pair % H);
  if (seq_of_token[t] < 0) return;
  const float* row = o + ((size_t)t * H + h) * Dv;
  float s = 0.f;
  for (int j = lane; j < Dv; j += WAVE) s = fmaf(row[j], row[j], s);
  s = wave_sum(s);
  const float inv = 1.f / sqrtf(s / (float)Dv + eps);
  for (int j = lane; j < Dv; j += WAVE) {
    const float g = fms_activate(gate[(size_t)t * ldg + (size_t)h * Dv + j], act);
    out[(size_t)t * ldo + (size_t)h * Dv + j] = from_f32<T>(row[j] * inv * to_f32(weight[j]) * g * out_scale);
  }
}

// --------------------------------------------------------------------------
extern "C" int fmsamd_delta_prepare(const float* proj, long ld, int col_b, const float* a, long lda, int col_a, const void* conv_w,
                                    int conv_dtype, int taps, const float* a_log, const float* dt_bias, float* conv_state,
                                    const int* seq_of_token, const int* slot_ids, float* qkv, float* beta, float* decay,
                                    int n_tokens, int heads, int kv_heads, int dim, int vdim, int per_channel, float q_scale,
                                    hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0,
              "delta_prepare: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, dim, vdim);
  FMS_REQUIRE(taps >= 1 && taps <= DELTA_MAX_TAPS, "delta_prepare: %d taps (1 to %d)", taps, DELTA_MAX_TAPS);
  const long C = 2L * kv_heads * dim + (long)heads * vdim;
  FMS_REQUIRE(ld >= C && col_b >= 0 && col_b + heads <= ld, "delta_prepare: rows of %ld for %ld channels", ld, C);
  FMS_REQUIRE(C * 4 <= 64 * 1024, "delta_prepare: %ld channels do not fit one block's LDS", C);
  FMS_REQUIRE(col_a >= 0 && col_a + heads * (per_channel ? dim : 1) <= lda, "delta_prepare: the decay's columns leave its rows");
  const size_t lds = (size_t)C * sizeof(float);
#define FMS_PREP(W)                                                                                                   \
  delta_prepare_kernel<W><<<n_tokens, 256, lds, stream>>>(proj, ld, col_b, a, lda, col_a, (const W*)conv_w, taps, a_log, \
                                                          dt_bias, conv_state, seq_of_token, slot_ids, qkv, beta, decay, \
                                                          heads, kv_heads, dim, vdim, per_channel, q_scale)
  if (conv_dtype == FMS_F32) FMS_PREP(float);
  else if (conv_dtype == FMS_BF16) FMS_PREP(bf16);
  else FMS_REQUIRE(false, "delta_prepare: unknown dtype %d", conv_dtype);
#undef FMS_PREP
  FMS_LAUNCH_CHECK("delta_prepare");
  if (taps > 1) {
    conv_state_kernel<<<n_tokens, 256, 0, stream>>>(proj, ld, taps, conv_state, seq_of_token, slot_ids, n_tokens, (int)C);
    FMS_LAUNCH_CHECK("conv_state");
  }
  return 0;
}

extern "C" int fmsamd_delta_rule(const float* qkv, const float* beta, const float* decay, float* state, float* out,
                                 const int* seq_starts, const int* seq_of_token, const int* slot_ids, int n_seqs, int heads,
                                 int kv_heads, int dim, int vdim, int per_channel, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  FMS_REQUIRE(n_seqs > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0,
              "delta_rule: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, dim, vdim);
  FMS_REQUIRE(dim <= 16 * DELTA_PARTS, "delta_rule: %d key channels (at most %d)", dim, 16 * DELTA_PARTS);
  FMS_REQUIRE(heads <= 65535 && ceil_div(vdim, DELTA_COLS) <= 65535, "delta_rule: too many heads or value channels for one launch");
  DeltaArgs a{qkv, beta, decay, state, out, seq_starts, seq_of_token, slot_ids, heads, kv_heads, dim, vdim, per_channel};
  const dim3 grid(n_seqs, heads, ceil_div(vdim, DELTA_COLS));
  if (dim <= 2 * DELTA_PARTS) delta_rule_kernel<2, 16><<<grid, WAVE, 0, stream>>>(a);
  else if (dim <= 4 * DELTA_PARTS) delta_rule_kernel<4, 16><<<grid, WAVE, 0, stream>>>(a);
  else if (dim <= 8 * DELTA_PARTS) delta_rule_kernel<8, 16><<<grid, WAVE, 0, stream>>>(a);
  else delta_rule_kernel<16, 8><<<grid, WAVE, 0, stream>>>(a);
  FMS_LAUNCH_CHECK("delta_rule");
  return 0;
}

extern "C" int fmsamd_gated_head_norm(const float* o, const float* gate, long ldg, const void* weight, int weight_dtype, float eps,
                                      int act, float out_scale, void* out, int out_dtype, long ldo, const int* seq_of_token,
                                      int n_tokens, int heads, int vdim, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && heads > 0 && vdim > 0 && ldg >= (long)heads * vdim && ldo >= (long)heads * vdim,
              "gated_head_norm: bad sizes heads=%d vdim=%d", heads, vdim);
  FMS_REQUIRE(act >= 0 && act <= FMS_ACT_LAST, "gated_head_norm: unknown activation %d", act);
  const int blocks = ceil_div((long)n_tokens * heads, 4);
#define FMS_GHN(T, W)                                                                                                          \
  gated_head_norm_kernel<T, W><<<blocks, 256, 0, stream>>>(o, gate, ldg, (const W*)weight, eps, act, out_scale, (T*)out, ldo, \
                                                           seq_of_token, n_tokens, heads, vdim)
  if (out_dtype == FMS_F32 && weight_dtype == FMS_F32) FMS_GHN(float, float);
  else if (out_dtype == FMS_BF16 && weight_dtype == FMS_F32) FMS_GHN(bf16, float);
  else if (out_dtype == FMS_BF16 && weight_dtype == FMS_BF16) FMS_GHN(bf16, bf16);
  else if (out_dtype == FMS_F32 && weight_dtype == FMS_BF16) FMS_GHN(float, bf16);
  else FMS_REQUIRE(false, "gated_head_norm: unknown dtypes %d, %d", out_dtype, weight_dtype);
#undef FMS_GHN
  FMS_LAUNCH_CHECK("gated_head_norm");
  return 0;
}
