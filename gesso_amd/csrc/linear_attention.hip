// Linear attention through a fading matrix state, and the norm and gate of its output.
//
// Per sequence and head a state S (n x m, float32, in the request's slot) is advanced token by token:
//
//   S <- decay_h S + k_t v_t^T,   o_t = S^T q_t
//
// q_t, k_t (n values) and v_t (m values) are columns of a row buffer x (T, ld): q of head h at [oq + h n, ...), k at
// [ok + h n, ...), v at [ov + h m, ...).  On their way in they may be activated (silu), q and k may be turned by the
// token's position (the first rd features of a head, feature i with i + rd/2, cos and sin from tables made on the
// host), and k may be scaled, all in float32: what enters the state is never rounded to the activation type again.
//
// linear_attention_scan: one block per (sequence, head, tile of 64 value columns); the columns of S are independent
// of each other, so wide values share out over blocks.  Thread (rg, jl) = (tid & 3, tid >> 2) holds the state's rows
// rg, rg + 4, ... of column jl in registers; the four partial sums of a column's output are neighbours in a
// wavefront.  A step's tokens come through LDS eight at a time.  The sums run in one fixed order per output, whatever
// the step's cut: a sequence fed whole, in portions or token by token leaves the same state and outputs, bit for bit.
// A step of single tokens is the same kernel with one token a block.  With `below` > 0 only the sequences that bring
// fewer tokens than that are taken: the longer ones go to the kernel on the matrix cores (linear_attention_mfma.hip).
//
// gated_outnorm: the heads' outputs of a token, normed in float32 (all heads as one row with a weight, or each head by
// its own root mean square, no weight) and multiplied by sigmoid or silu of a gate row.
#include "common.h"

#define LA_TB 8          // tokens staged at once
#define LA_COLS 64       // value columns a block

__device__ __forceinline__ float la_act(float z, int act) { return act ? z / (1.0f + expf(-z)) : z; }

template <typename TI, int RMAX>
__global__ void __launch_bounds__(256)
linear_attention_scan_kernel(const TI* __restrict__ x, int ld, int oq, int ok, int ov, int act,
                             const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rd, float key_scale,
                             const float* __restrict__ decay, float* __restrict__ state,
                             const int* __restrict__ q_start, const int* __restrict__ slots,
                             const int* __restrict__ positions, float* __restrict__ out, int H, int n, int m,
                             int below) {
  constexpr int NMAX = 4 * RMAX;
  __shared__ float qs[LA_TB][NMAX];
  __shared__ float ks[LA_TB][NMAX];
  __shared__ float vs[LA_TB][LA_COLS];
  const int seq = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * LA_COLS;
  const int tid = threadIdx.x, rg = tid & 3, jl = tid >> 2, j = j0 + jl;
  const int t0 = q_start[seq], t1 = q_start[seq + 1];
  if (t1 <= t0 || (below > 0 && t1 - t0 >= below)) return;      // (longer sequences are another kernel's)
  const float d = decay[h];
  float* S = state + (((size_t)slots[seq] * H + h) * n) * m;
  float s[RMAX];
#pragma unroll
  for (int r = 0; r < RMAX; ++r) {
    const int i = rg + 4 * r;
    s[r] = (i < n && j < m) ? S[(size_t)i * m + j] : 0.f;
  }
  const int half = rd >> 1;
  for (int tb = t0; tb < t1; tb += LA_TB) {
    const int nb = t1 - tb < LA_TB ? t1 - tb : LA_TB;
    __syncthreads();                                   // the batch before has been read
    for (int idx = tid; idx < nb * n; idx += 256) {
      const int tt = idx / n, i = idx - tt * n;
      const TI* row = x + (size_t)(tb + tt) * ld;
      float qv = la_act(to_f32(row[oq + h * n + i]), act);
      float kv = la_act(to_f32(row[ok + h * n + i]), act);
      if (i < rd) {
        const bool low = i < half;
        const int p = low ? i : i - half, other = low ? i + half : i - half;
        const size_t at = (size_t)positions[tb + tt] * half + p;
        const float c = cos_t[at], sn = sin_t[at];
        const float qo = la_act(to_f32(row[oq + h * n + other]), act);
        const float ko = la_act(to_f32(row[ok + h * n + other]), act);
        // (u, v) -> (u cos - v sin, v cos + u sin)
        qv = low ? qv * c - qo * sn : qv * c + qo * sn;
        kv = low ? kv * c - ko * sn : kv * c + ko * sn;
      }
      qs[tt][i] = qv;
      ks[tt][i] = kv * key_scale;
    }
    for (int idx = tid; idx < nb * LA_COLS; idx += 256) {
      const int tt = idx / LA_COLS, c = idx - tt * LA_COLS;
      vs[tt][c] = j0 + c < m ? la_act(to_f32(x[(size_t)(tb + tt) * ld + ov + h * m + j0 + c]), act) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nb; ++tt) {
      const float vj = vs[tt][jl];
      float part = 0.f;
#pragma unroll
      for (int r = 0; r < RMAX; ++r) {
        const int i = rg + 4 * r;
        if (i < n) {
          s[r] = fmaf(ks[tt][i], vj, d * s[r]);
          part = fmaf(s[r], qs[tt][i], part);
        }
      }
      part += __shfl_xor(part, 1, 64);
      part += __shfl_xor(part, 2, 64);
      if (rg == 0 && j < m) out[((size_t)(tb + tt) * H + h) * m + j] = part;
    }
  }
#pragma unroll
  for (int r = 0; r < RMAX; ++r) {
    const int i = rg + 4 * r;
    if (i < n && j < m) S[(size_t)i * m + j] = s[r];
  }
}

extern "C" int gs_linear_attention_scan(const void* x, int dtype, int ld, int oq, int ok, int ov, int act,
                                        const float* cos_t, const float* sin_t, int rd, int max_position,
                                        float key_scale, const float* decay, float* state, const int* q_start,
                                        const int* slots, const int* positions, float* out, int nseq, int H, int n,
                                        int m, int below, hipStream_t stream) {
  GS_REQUIRE(nseq >= 0 && H > 0 && n > 0 && m > 0, "linear_attention: bad sizes nseq=%d H=%d n=%d m=%d", nseq, H, n, m);
  GS_REQUIRE(n <= 512, "linear_attention: keys of %d features, the kernel holds up to 512", n);
  GS_REQUIRE(H <= 65535 && (m + LA_COLS - 1) / LA_COLS <= 65535, "linear_attention: too many heads or value columns");
  GS_REQUIRE(rd >= 0 && rd <= n && rd % 2 == 0, "linear_attention: %d turned features of %d", rd, n);
  GS_REQUIRE(rd == 0 || (cos_t && sin_t && max_position > 0), "linear_attention: rotation without a table");
  GS_REQUIRE(oq >= 0 && ok >= 0 && ov >= 0 && oq + H * n <= ld && ok + H * n <= ld && ov + H * m <= ld,
             "linear_attention: q, k or v lie outside the rows of %d", ld);
  GS_REQUIRE(act == 0 || act == 1, "linear_attention: unknown activation %d", act);
  if (nseq == 0) return 0;
  dim3 grid(nseq, H, (m + LA_COLS - 1) / LA_COLS);
#define LA_RUN(TI, R)                                                                                                \
  linear_attention_scan_kernel<TI, R><<<grid, 256, 0, stream>>>((const TI*)x, ld, oq, ok, ov, act, cos_t, sin_t, rd, \
                                                                key_scale, decay, state, q_start, slots, positions,  \
                                                                out, H, n, m, below)
#define LA_RUN_T(TI)                      \
  if (n <= 32) LA_RUN(TI, 8);             \
  else if (n <= 64) LA_RUN(TI, 16);       \
  else if (n <= 128) LA_RUN(TI, 32);      \
  else if (n <= 256) LA_RUN(TI, 64);      \
  else LA_RUN(TI, 128)
  if (dtype == GS_F32) {
    LA_RUN_T(float);
  } else if (dtype == GS_BF16) {
    LA_RUN_T(bf16);
  } else {
    GS_REQUIRE(false, "linear_attention: unknown dtype %d", dtype);
  }
#undef LA_RUN_T
#undef LA_RUN
  GS_LAUNCH_CHECK("linear_attention_scan");
  return 0;
}

// One block per token.  o (T, H m) float32; gate rows in a buffer (T, ldg) at column og.
//   joint: y = o / sqrt(mean over all H m values + eps) * w;   else, per head: y = o / sqrt(mean over the head's m + eps)
//   out = y * g(gate),  g = sigmoid (gate_act 0) or silu (1)
template <typename TI, typename TO>
__global__ void gated_outnorm_kernel(const float* __restrict__ o, const TI* __restrict__ gate, int ldg, int og,
                                     const float* __restrict__ w, float eps, int joint, int gate_act,
                                     TO* __restrict__ out, int H, int m) {
  __shared__ float red[17];
  const int t = blockIdx.x, W = H * m;
  const float* row = o + (size_t)t * W;
  const TI* g = gate + (size_t)t * ldg + og;
  TO* dst = out + (size_t)t * W;
  if (joint && (W & 7) == 0 && W <= 8 * 256 * 4 && aligned16(row) && aligned16(g) && aligned16(dst) && (!w || aligned16(w))) {
    // eight values a thread and turn, the row in registers between the two passes (rows up to 8192 values)
    float keep[4][8];
    float ss = 0.f;
    const int turns = (W / 8 + blockDim.x - 1) / blockDim.x;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = (u * blockDim.x + threadIdx.x) * 8;
      if (u < turns && c < W) {
        load8f(row + c, keep[u]);
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += keep[u][i] * keep[u][i];
      }
    }
    ss = block_sum(ss, red);
    const float inv = norm_inverse(ss, (float)W, eps);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = (u * blockDim.x + threadIdx.x) * 8;
      if (u < turns && c < W) {
        float z[8], w8[8], y[8];
        load8f(g + c, z);
        if (w) load8f(w + c, w8);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float sg = 1.0f / (1.0f + expf(-z[i]));
          y[i] = keep[u][i] * inv * (w ? w8[i] : 1.f) * (gate_act ? z[i] * sg : sg);
        }
        store8f(dst + c, y);
      }
    }
    return;
  }
  if (joint) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) ss += row[c] * row[c];
    ss = block_sum(ss, red);
    const float inv = norm_inverse(ss, (float)W, eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      const float z = to_f32(g[c]);
      const float sg = 1.0f / (1.0f + expf(-z));
      dst[c] = from_f32<TO>(row[c] * inv * (w ? w[c] : 1.f) * (gate_act ? z * sg : sg));
    }
    return;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int h = wave; h < H; h += nw) {
    float ss = 0.f;
    for (int c = lane; c < m; c += 64) ss += row[h * m + c] * row[h * m + c];
    ss = wave_sum(ss);
    const float inv = norm_inverse(ss, (float)m, eps);
    for (int c = lane; c < m; c += 64) {
      const float z = to_f32(g[h * m + c]);
      const float sg = 1.0f / (1.0f + expf(-z));
      dst[h * m + c] = from_f32<TO>(row[h * m + c] * inv * (w ? w[h * m + c] : 1.f) * (gate_act ? z * sg : sg));
    }
  }
}

extern "C" int gs_gated_outnorm(const float* o, const void* gate, int gate_dtype, int ldg, int og, const float* w,
                                float eps, int joint, int gate_act, void* out, int out_dtype, int T, int H, int m,
                                hipStream_t stream) {
  GS_REQUIRE(T >= 0 && H > 0 && m > 0, "gated_outnorm: bad sizes T=%d H=%d m=%d", T, H, m);
  GS_REQUIRE(eps > 0.f, "gated_outnorm: eps must be positive");
  GS_REQUIRE(og >= 0 && og + H * m <= ldg, "gated_outnorm: the gate lies outside the rows of %d", ldg);
  GS_REQUIRE(gate_dtype == out_dtype, "gated_outnorm: gate and result are of one type");
  if (T == 0) return 0;
  if (out_dtype == GS_F32)
    gated_outnorm_kernel<float, float><<<T, 256, 0, stream>>>(o, (const float*)gate, ldg, og, w, eps, joint, gate_act,
                                                               (float*)out, H, m);
  else if (out_dtype == GS_BF16)
    gated_outnorm_kernel<bf16, bf16><<<T, 256, 0, stream>>>(o, (const bf16*)gate, ldg, og, w, eps, joint, gate_act,
                                                             (bf16*)out, H, m);
  else
    GS_REQUIRE(false, "gated_outnorm: unknown dtype %d", out_dtype);
  GS_LAUNCH_CHECK("gated_outnorm");
  return 0;
}
