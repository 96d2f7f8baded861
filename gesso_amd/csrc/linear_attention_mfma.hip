// Linear attention through a fading matrix state for prompt portions, on the matrix cores.
//
// The same recurrence as linear_attention.hip (S <- decay S + k_t v_t^T, o_t = S^T q_t, per sequence and head), taken
// 32 tokens at a time.  With Q, K (32 x n) and V (32 x m) the rows of a run of L <= 32 tokens and S the state before it:
//
//   O  = diag(d^(t+1)) Q S  +  ((Q K^T) o D) V,     D[t][s] = d^(t-s) for s <= t, else 0
//   S' = d^L S + sum_s d^(L-1-s) k_s v_s^T
//
// One block per (sequence, head, 128 value columns), four wavefronts, each owning 32 of the columns: its slice of the
// state (transposed, 32 x n) stays in its accumulators from run to run.  Products are v_mfma_f32_32x32x16_bf16 with
// float32 sums.  What the design holds in 32 bits (activated and turned q and k, the decayed scores, the state, the
// decayed keys) enters the products as two bfloat16 terms, the value's rounding and the rounding of what is left, and
// each product is three (hi hi + hi lo + lo hi): sixteen bits of every operand, the sums in float32.  Values as they
// come from their product are bfloat16 already and enter as one term; activated values as two, like the rest.  Powers
// of the decay come from a table made by repeated multiplication.
//
// The scores are computed transposed (rows s, columns t), which leaves them, in a lane's registers, in the order in
// which the next product takes its first operand, but for a permutation of the 16 inner indices of a step: slot q of
// lane half hf stands for s = 16 step + 8 (q / 4) + 4 hf + q % 4; the value operand is read in the same order (two
// 8-byte reads).  No trip of the scores through LDS, no wait between the two products.
//
// Sequences shorter than `min_len` tokens are left alone (the token-by-token kernel takes them).
//
// One block a (sequence, head) walks the runs one after the other, which leaves most of the chip idle when a step
// brings few long portions.  Then the portions are cut into segments of `seg_len` tokens and three launches do the
// work (MODE): (1) every segment by a block of its own, from the request's state (the first segment) or from an empty
// one, its outputs stored and its last state left in a workspace; (2) a light kernel goes through a sequence's
// segments in order, S_start[p + 1] = d^len(p) S_start[p] + G[p], leaves every segment's first state in the workspace
// and the last state in the request's slot; (3) every segment but the first adds what its first state gives its
// tokens, d^(t + 1) q_t S_start, the first of the two terms of O above, with the state's decay from run to run kept
// as one factor.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 lm_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 lm_bf16x4_t;
typedef __attribute__((ext_vector_type(16))) float lm_f32x16_t;

constexpr int LM_C = 32;          // tokens a run
constexpr int LM_MTB = 128;       // value columns a block
constexpr int LM_LDT = LM_C + 8;  // elements per LDS row of the transposed operands

// silu by the hardware's exponential and reciprocal (each good to a unit in the last place of float32)
__device__ __forceinline__ float lm_act(float z, int act) {
  return act ? z * __builtin_amdgcn_rcpf(1.0f + __expf(-z)) : z;
}

__device__ __forceinline__ void lm_split(float v, uint16_t& hi, uint16_t& lo) {
  const bf16 h = f32_to_bf16(v);
  hi = h.x;
  lo = f32_to_bf16(v - to_f32(h)).x;
}

template <int NT, bool VEC, int MODE>
__global__ __launch_bounds__(256) void linear_attention_chunk_kernel(
    const bf16* __restrict__ x, int ld, int oq, int ok, int ov, int act, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int rd, float key_scale, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ q_start, const int* __restrict__ slots,
    const int* __restrict__ positions, float* __restrict__ out, int H, int n, int m, int min_len,
    float* __restrict__ ws, int maxseg, int seg_len) {
  constexpr int NP = 32 * NT, LDQ = NP + 8;
  extern __shared__ __align__(16) uint16_t lm_lds[];
  uint16_t* Qh = lm_lds;  // [32][LDQ] each
  uint16_t* Ql = Qh + LM_C * LDQ;
  uint16_t* Kh = Ql + LM_C * LDQ;
  uint16_t* Kl = Kh + LM_C * LDQ;
  uint16_t* KTh = Kl + LM_C * LDQ;  // [NP][LDT] each: decayed keys, transposed
  uint16_t* KTl = KTh + NP * LM_LDT;
  uint16_t* VT = KTl + NP * LM_LDT;      // [MTB][LDT]: values, transposed
  uint16_t* VTl = VT + LM_MTB * LM_LDT;  // the same: what the rounding of activated values left
  uint16_t* STh = VTl + LM_MTB * LM_LDT;  // [MTB][LDQ] each: the state, transposed
  uint16_t* STl = STh + LM_MTB * LDQ;
  __shared__ float pw[LM_C + 1];

  const int seq = MODE == 0 ? blockIdx.x : blockIdx.x / maxseg, seg = MODE == 0 ? 0 : blockIdx.x % maxseg;
  const int h = blockIdx.y, j0 = blockIdx.z * LM_MTB;
  const int ts = q_start[seq];            // the sequence's first row of this step
  int t0 = ts, t1 = q_start[seq + 1];
  if (t1 - t0 < min_len || t1 <= t0) return;
  if (MODE != 0) {
    if (MODE == 2 && seg == 0) return;    // the first segment started from the true state
    t0 = ts + seg * seg_len;
    if (t0 >= t1) return;
    t1 = t1 < t0 + seg_len ? t1 : t0 + seg_len;
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
  const int jw = wave * 32;
  const bool live = j0 + jw < m;      // a wavefront whose columns all lie beyond m only helps staging
  const float d = decay[h];
  // where the state comes from and goes to: the request's slot, or the segment's place in the workspace
  float* W = MODE == 0 ? nullptr : ws + ((((size_t)seq * maxseg + seg) * H + h) * n) * m;
  float* S = (MODE == 0 || (MODE == 1 && seg == 0)) ? state + (((size_t)slots[seq] * H + h) * n) * m : W;
  const bool empty = MODE == 1 && seg > 0;
  if (tid == 0) {
    float p = 1.f;
    for (int e = 0; e <= LM_C; ++e) {
      pw[e] = p;
      p *= d;
    }
  }
  lm_f32x16_t acc_s[NT];
#pragma unroll
  for (int it = 0; it < NT; ++it)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int i = it * 32 + l32, j = j0 + jw + 8 * (e / 4) + 4 * half + e % 4;
      acc_s[it][e] = (!empty && i < n && j < m) ? S[(size_t)i * m + j] : 0.f;
    }
  const int hr = rd >> 1;
  float cum = 1.f;        // MODE 2: the state's decay over the runs gone by

  // VEC: a run's rows come as 16-byte pieces (eight features of one token), all of a thread's pieces asked for at once
  // and, from the second run on, while the run before is still being computed.  Piece u of a thread: token
  // (tid + 256 u) % 32, features 8 ((tid + 256 u) / 32) ... (neighbouring lanes hold neighbouring tokens, so that the
  // transposed stores into LDS fall side by side); a piece's partner in the turn is a whole piece too (rd / 2 a
  // multiple of eight).  Values: piece (tid + 256 u) % 32 -> token, / 32 -> eight columns.
  constexpr int UQ = (LM_C * NP / 8 + 255) / 256, UV = LM_C * LM_MTB / 8 / 256;
  uint4 rq[UQ], rk[UQ], rqo[UQ], rko[UQ], rv[UV];
  const int pos0 = positions[ts];
  auto fetch = [&](int tb, int nb) {
    if constexpr (VEC) {
#pragma unroll
      for (int u = 0; u < UQ; ++u) {
        const int piece = tid + 256 * u, t = piece % LM_C, i = (piece / LM_C) * 8;
        rq[u] = rk[u] = rqo[u] = rko[u] = make_uint4(0, 0, 0, 0);
        if (t < nb && i < n) {
          const bf16* row = x + (size_t)(tb + t) * ld;
          rq[u] = *reinterpret_cast<const uint4*>(row + oq + h * n + i);
          if (MODE != 2) rk[u] = *reinterpret_cast<const uint4*>(row + ok + h * n + i);
          if (i < rd) {
            const int other = i < hr ? i + hr : i - hr;
            rqo[u] = *reinterpret_cast<const uint4*>(row + oq + h * n + other);
            if (MODE != 2) rko[u] = *reinterpret_cast<const uint4*>(row + ok + h * n + other);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < UV; ++u) {
        const int piece = tid + 256 * u, t = piece % LM_C, c = (piece / LM_C) * 8;
        rv[u] = make_uint4(0, 0, 0, 0);
        if (MODE != 2 && t < nb && j0 + c < m)
          rv[u] = *reinterpret_cast<const uint4*>(x + (size_t)(tb + t) * ld + ov + h * m + j0 + c);
      }
    }
  };
  auto eight = [](const uint4& w, float* v) {
    const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[2 * e] = __uint_as_float(ww[e] << 16);
      v[2 * e + 1] = __uint_as_float(ww[e] & 0xffff0000u);
    }
  };
  if (t1 > t0) fetch(t0, t1 - t0 < LM_C ? t1 - t0 : LM_C);

  for (int tb = t0; tb < t1; tb += LM_C) {
    const int nb = t1 - tb < LM_C ? t1 - tb : LM_C;
    __syncthreads();  // the run before has been read (and, the first time, the table of powers is there)
    if constexpr (VEC) {
#pragma unroll
      for (int u = 0; u < UQ; ++u) {
        const int piece = tid + 256 * u, t = piece % LM_C, i = (piece / LM_C) * 8;
        if (i >= NP) continue;
        float q8[8], k8[8], qo[8], ko[8];
        eight(rq[u], q8);
        eight(rk[u], k8);
        eight(rqo[u], qo);
        eight(rko[u], ko);
        const bool turned = t < nb && i < rd, low = i < hr;
        float c8[8], s8[8];
        if (turned) {
          const float* cr = cos_t + (size_t)(pos0 + tb - ts + t) * hr + (low ? i : i - hr);
          const float* sr = sin_t + (size_t)(pos0 + tb - ts + t) * hr + (low ? i : i - hr);
          load8f(cr, c8);
          load8f(sr, s8);
        }
        const float kdec = t < nb ? pw[nb - 1 - t] : 0.f;
        uint16_t qh[8], ql[8], kh[8], kl[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float qv = lm_act(q8[e], act), kv = lm_act(k8[e], act);
          if (turned) {
            const float qp = lm_act(qo[e], act), kp = lm_act(ko[e], act);
            qv = low ? qv * c8[e] - qp * s8[e] : qv * c8[e] + qp * s8[e];
            kv = low ? kv * c8[e] - kp * s8[e] : kv * c8[e] + kp * s8[e];
          }
          kv *= key_scale;
          lm_split(qv, qh[e], ql[e]);
          if constexpr (MODE != 2) {
            lm_split(kv, kh[e], kl[e]);
            lm_split(kv * kdec, KTh[(i + e) * LM_LDT + t], KTl[(i + e) * LM_LDT + t]);
          }
        }
        auto pack = [](const uint16_t* v) {
          return make_uint4(v[0] | ((uint32_t)v[1] << 16), v[2] | ((uint32_t)v[3] << 16), v[4] | ((uint32_t)v[5] << 16),
                            v[6] | ((uint32_t)v[7] << 16));
        };
        *reinterpret_cast<uint4*>(Qh + t * LDQ + i) = pack(qh);
        *reinterpret_cast<uint4*>(Ql + t * LDQ + i) = pack(ql);
        if constexpr (MODE != 2) {     // (the pass that adds a first state's term needs the queries alone)
          *reinterpret_cast<uint4*>(Kh + t * LDQ + i) = pack(kh);
          *reinterpret_cast<uint4*>(Kl + t * LDQ + i) = pack(kl);
        }
      }
#pragma unroll
      for (int u = 0; u < (MODE == 2 ? 0 : UV); ++u) {
        const int piece = tid + 256 * u, t = piece % LM_C, c = (piece / LM_C) * 8;
        float v8[8];
        eight(rv[u], v8);
#pragma unroll
        for (int e = 0; e < 8; ++e) lm_split(lm_act(v8[e], act), VT[(c + e) * LM_LDT + t], VTl[(c + e) * LM_LDT + t]);
      }
    } else {
      for (int idx = tid; idx < LM_C * NP; idx += 256) {
        const int t = idx / NP, i = idx - t * NP;
        float qv = 0.f, kv = 0.f;
        if (t < nb && i < n) {
          const bf16* row = x + (size_t)(tb + t) * ld;
          qv = lm_act(to_f32(row[oq + h * n + i]), act);
          kv = lm_act(to_f32(row[ok + h * n + i]), act);
          if (i < rd) {
            const bool low = i < hr;
            const int p = low ? i : i - hr, other = low ? i + hr : i - hr;
            const size_t at = (size_t)positions[tb + t] * hr + p;
            const float c = cos_t[at], sn = sin_t[at];
            const float qo = lm_act(to_f32(row[oq + h * n + other]), act);
            const float ko = lm_act(to_f32(row[ok + h * n + other]), act);
            qv = low ? qv * c - qo * sn : qv * c + qo * sn;
            kv = low ? kv * c - ko * sn : kv * c + ko * sn;
          }
          kv *= key_scale;
        }
        lm_split(qv, Qh[t * LDQ + i], Ql[t * LDQ + i]);
        lm_split(kv, Kh[t * LDQ + i], Kl[t * LDQ + i]);
        const float kd = t < nb ? kv * pw[nb - 1 - t] : 0.f;
        lm_split(kd, KTh[i * LM_LDT + t], KTl[i * LM_LDT + t]);
      }
      for (int idx = tid; idx < LM_C * LM_MTB; idx += 256) {
        const int t = idx / LM_MTB, c = idx - t * LM_MTB;
        const int j = j0 + c;
        const float v = (t < nb && j < m) ? lm_act(to_f32(x[(size_t)(tb + t) * ld + ov + h * m + j]), act) : 0.f;
        lm_split(v, VT[c * LM_LDT + t], VTl[c * LM_LDT + t]);
      }
    }
    if (live && (MODE != 2 || tb == t0)) {
#pragma unroll
      for (int it = 0; it < NT; ++it)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int jj = jw + 8 * (e / 4) + 4 * half + e % 4, ii = it * 32 + l32;
          lm_split(acc_s[it][e], STh[jj * LDQ + ii], STl[jj * LDQ + ii]);
        }
    }
    __syncthreads();
    if (tb + LM_C < t1) fetch(tb + LM_C, t1 - tb - LM_C < LM_C ? t1 - tb - LM_C : LM_C);   // the next run's rows, meanwhile
    if (!live) continue;

    if constexpr (MODE == 2) {
      lm_f32x16_t o2;
#pragma unroll
      for (int e = 0; e < 16; ++e) o2[e] = 0.f;
      const int ro2 = l32 * LDQ + half * 8, so2 = (jw + l32) * LDQ + half * 8;
#pragma unroll
      for (int ks = 0; ks < NP / 16; ++ks) {
        const lm_bf16x8_t qh8 = *reinterpret_cast<const lm_bf16x8_t*>(Qh + ro2 + ks * 16);
        const lm_bf16x8_t ql8 = *reinterpret_cast<const lm_bf16x8_t*>(Ql + ro2 + ks * 16);
        const lm_bf16x8_t sh8 = *reinterpret_cast<const lm_bf16x8_t*>(STh + so2 + ks * 16);
        const lm_bf16x8_t sl8 = *reinterpret_cast<const lm_bf16x8_t*>(STl + so2 + ks * 16);
        o2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qh8, sh8, o2, 0, 0, 0);
        o2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qh8, sl8, o2, 0, 0, 0);
        o2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ql8, sh8, o2, 0, 0, 0);
      }
      const int j2 = j0 + jw + l32;
      if (j2 < m) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int t = 8 * (e / 4) + 4 * half + e % 4;
          if (t < nb) out[((size_t)(tb + t) * H + h) * m + j2] += o2[e] * (pw[t + 1] * cum);
        }
      }
      cum *= pw[nb];
      continue;
    }
    // scores, transposed: rows s, columns t
    // (two accumulators in turn: a product that waits for the one before it idles the pipe for its whole latency)
    lm_f32x16_t at, at2;
#pragma unroll
    for (int e = 0; e < 16; ++e) at[e] = at2[e] = 0.f;
    const int ro = l32 * LDQ + half * 8;
#pragma unroll
    for (int ks = 0; ks < NP / 16; ++ks) {
      const lm_bf16x8_t kh8 = *reinterpret_cast<const lm_bf16x8_t*>(Kh + ro + ks * 16);
      const lm_bf16x8_t kl8 = *reinterpret_cast<const lm_bf16x8_t*>(Kl + ro + ks * 16);
      const lm_bf16x8_t qh8 = *reinterpret_cast<const lm_bf16x8_t*>(Qh + ro + ks * 16);
      const lm_bf16x8_t ql8 = *reinterpret_cast<const lm_bf16x8_t*>(Ql + ro + ks * 16);
      at = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kh8, qh8, at, 0, 0, 0);
      at2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kh8, ql8, at2, 0, 0, 0);
      at2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kl8, qh8, at2, 0, 0, 0);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) at[e] += at2[e];
    // this lane: query t = l32, keys s(e); the causal rule and the decay between the two; as operands of the next product
    lm_bf16x8_t ah[2], al[2];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int s = 8 * (e / 4) + 4 * half + e % 4;
      const float a = s <= l32 ? at[e] * pw[l32 - s] : 0.f;
      const bf16 hi = f32_to_bf16(a);
      ah[e / 8][e % 8] = __builtin_bit_cast(__bf16, hi.x);
      al[e / 8][e % 8] = __builtin_bit_cast(__bf16, f32_to_bf16(a - to_f32(hi)).x);
    }
    // what the state before the run gives: rows t, columns j, then each row times d^(t+1)
    lm_f32x16_t o, ob;
#pragma unroll
    for (int e = 0; e < 16; ++e) o[e] = ob[e] = 0.f;
    const int so = (jw + l32) * LDQ + half * 8;
#pragma unroll
    for (int ks = 0; ks < NP / 16; ++ks) {
      const lm_bf16x8_t qh8 = *reinterpret_cast<const lm_bf16x8_t*>(Qh + ro + ks * 16);
      const lm_bf16x8_t ql8 = *reinterpret_cast<const lm_bf16x8_t*>(Ql + ro + ks * 16);
      const lm_bf16x8_t sh8 = *reinterpret_cast<const lm_bf16x8_t*>(STh + so + ks * 16);
      const lm_bf16x8_t sl8 = *reinterpret_cast<const lm_bf16x8_t*>(STl + so + ks * 16);
      o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qh8, sh8, o, 0, 0, 0);
      ob = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qh8, sl8, ob, 0, 0, 0);
      ob = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ql8, sh8, ob, 0, 0, 0);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) o[e] = (o[e] + ob[e]) * pw[8 * (e / 4) + 4 * half + e % 4 + 1];
    // what the run's own tokens give
    const int vo = (jw + l32) * LM_LDT;
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2) {
      const lm_bf16x4_t v0 = *reinterpret_cast<const lm_bf16x4_t*>(VT + vo + 16 * k2 + 4 * half);
      const lm_bf16x4_t v1 = *reinterpret_cast<const lm_bf16x4_t*>(VT + vo + 16 * k2 + 8 + 4 * half);
      lm_bf16x8_t v8;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        v8[q] = v0[q];
        v8[4 + q] = v1[q];
      }
      o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[k2], v8, o, 0, 0, 0);
      o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[k2], v8, o, 0, 0, 0);
      if (act) {      // activated values have a second term
        const lm_bf16x4_t w0 = *reinterpret_cast<const lm_bf16x4_t*>(VTl + vo + 16 * k2 + 4 * half);
        const lm_bf16x4_t w1 = *reinterpret_cast<const lm_bf16x4_t*>(VTl + vo + 16 * k2 + 8 + 4 * half);
        lm_bf16x8_t w8;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          w8[q] = w0[q];
          w8[4 + q] = w1[q];
        }
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[k2], w8, o, 0, 0, 0);
      }
    }
    {
      const int j = j0 + jw + l32;
      if (j < m) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int t = 8 * (e / 4) + 4 * half + e % 4;
          if (t < nb) out[((size_t)(tb + t) * H + h) * m + j] = o[e];
        }
      }
    }
    // the state after the run: rows j, columns i
    const float dl = pw[nb];
#pragma unroll
    for (int it = 0; it < NT; ++it) {
#pragma unroll
      for (int e = 0; e < 16; ++e) acc_s[it][e] *= dl;
#pragma unroll
      for (int k2 = 0; k2 < 2; ++k2) {
        const lm_bf16x8_t v8 = *reinterpret_cast<const lm_bf16x8_t*>(VT + vo + 16 * k2 + 8 * half);
        const int ko = (it * 32 + l32) * LM_LDT + 16 * k2 + 8 * half;
        const lm_bf16x8_t kh8 = *reinterpret_cast<const lm_bf16x8_t*>(KTh + ko);
        const lm_bf16x8_t kl8 = *reinterpret_cast<const lm_bf16x8_t*>(KTl + ko);
        acc_s[it] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v8, kh8, acc_s[it], 0, 0, 0);
        acc_s[it] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v8, kl8, acc_s[it], 0, 0, 0);
        if (act) {
          const lm_bf16x8_t w8 = *reinterpret_cast<const lm_bf16x8_t*>(VTl + vo + 16 * k2 + 8 * half);
          acc_s[it] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w8, kh8, acc_s[it], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int it = 0; it < NT; ++it)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int i = it * 32 + l32, j = j0 + jw + 8 * (e / 4) + 4 * half + e % 4;
      if (MODE != 2 && i < n && j < m) (MODE == 0 ? S : W)[(size_t)i * m + j] = acc_s[it][e];
    }
}

// Pass (2) of the three: one thread per (sequence, head, element of the state), on its own through the segments.
__global__ void linear_attention_combine_kernel(const float* __restrict__ decay, float* __restrict__ state,
                                                const int* __restrict__ q_start, const int* __restrict__ slots,
                                                float* __restrict__ ws, int H, int n, int m, int min_len, int maxseg,
                                                int seg_len) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int len = q_start[seq + 1] - q_start[seq];
  if (len < min_len || len <= 0) return;
  const int nseg = (len + seg_len - 1) / seg_len;
  const float d = decay[h];
  float dfull = 1.f, dlast = 1.f;                     // d^seg_len and d^(the last segment's length), as the table's powers
  const int last = len - (nseg - 1) * seg_len;
  for (int e = 0; e < seg_len; ++e) {
    dfull *= d;
    if (e < last) dlast *= d;
  }
  const size_t per = (size_t)n * m;
  float* S = state + ((size_t)slots[seq] * H + h) * per;
  const size_t idx = (size_t)blockIdx.z * blockDim.x + threadIdx.x;
  if (idx < per) {
    float cur = ws[(((size_t)seq * maxseg) * H + h) * per + idx];
    for (int p = 1; p < nseg; ++p) {
      float* g = ws + (((size_t)seq * maxseg + p) * H + h) * per + idx;
      const float own = *g;
      *g = cur;                                       // the state the segment starts from
      cur = (p == nseg - 1 ? dlast : dfull) * cur + own;
    }
    S[idx] = cur;
  }
}

template <int NT, bool VEC, int MODE>
static void lm_launch(dim3 grid, hipStream_t stream, const bf16* x, int ld, int oq, int ok, int ov, int act,
                      const float* cos_t, const float* sin_t, int rd, float key_scale, const float* decay, float* state,
                      const int* q_start, const int* slots, const int* positions, float* out, int H, int n, int m,
                      int min_len, float* ws, int maxseg, int seg_len) {
  constexpr int NP = 32 * NT, LDQ = NP + 8;
  const size_t lds = (size_t)(4 * LM_C * LDQ + 2 * NP * LM_LDT + 2 * LM_MTB * LM_LDT + 2 * LM_MTB * LDQ) * sizeof(uint16_t);
  // more than the default limit of dynamic LDS: asked for once per kernel
  static const hipError_t asked = hipFuncSetAttribute(reinterpret_cast<const void*>(&linear_attention_chunk_kernel<NT, VEC, MODE>),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  (void)asked;
  linear_attention_chunk_kernel<NT, VEC, MODE><<<grid, 256, lds, stream>>>(x, ld, oq, ok, ov, act, cos_t, sin_t, rd,
                                                                           key_scale, decay, state, q_start, slots,
                                                                           positions, out, H, n, m, min_len, ws, maxseg,
                                                                           seg_len);
}

extern "C" int gs_linear_attention_chunks(const void* x, int ld, int oq, int ok, int ov, int act, const float* cos_t,
                                          const float* sin_t, int rd, int max_position, float key_scale,
                                          const float* decay, float* state, const int* q_start, const int* slots,
                                          const int* positions, float* out, int nseq, int H, int n, int m, int min_len,
                                          float* ws, int maxseg, int seg_len, hipStream_t stream) {
  GS_REQUIRE(maxseg >= 0 && (maxseg == 0 || (ws && seg_len > 0 && seg_len % LM_C == 0)),
             "linear_attention_chunks: segments of %d tokens (whole runs of %d) with a workspace", seg_len, LM_C);
  GS_REQUIRE(maxseg == 0 || (long)nseq * maxseg <= 0x7fffffffL, "linear_attention_chunks: too many segments");
  GS_REQUIRE(nseq >= 0 && H > 0 && n > 0 && m > 0, "linear_attention_chunks: bad sizes nseq=%d H=%d n=%d m=%d", nseq, H, n, m);
  GS_REQUIRE(n <= 128, "linear_attention_chunks: keys of %d features, the kernel holds up to 128", n);
  GS_REQUIRE(H <= 65535 && (m + LM_MTB - 1) / LM_MTB <= 65535, "linear_attention_chunks: too many heads or value columns");
  GS_REQUIRE(rd >= 0 && rd <= n && rd % 2 == 0, "linear_attention_chunks: %d turned features of %d", rd, n);
  GS_REQUIRE(rd == 0 || (cos_t && sin_t && max_position > 0), "linear_attention_chunks: rotation without a table");
  GS_REQUIRE(oq >= 0 && ok >= 0 && ov >= 0 && oq + H * n <= ld && ok + H * n <= ld && ov + H * m <= ld,
             "linear_attention_chunks: q, k or v lie outside the rows of %d", ld);
  GS_REQUIRE(act == 0 || act == 1, "linear_attention_chunks: unknown activation %d", act);
  if (nseq == 0) return 0;
  dim3 grid(maxseg > 0 ? nseq * maxseg : nseq, H, (m + LM_MTB - 1) / LM_MTB);
  // rows as 16-byte pieces where every piece is whole and aligned, a turn's partner piece included
  const bool vec = n % 8 == 0 && m % 8 == 0 && ld % 8 == 0 && oq % 8 == 0 && ok % 8 == 0 && ov % 8 == 0 && rd % 16 == 0 &&
                   ((uintptr_t)x & 15) == 0 && ((uintptr_t)cos_t & 15) == 0 && ((uintptr_t)sin_t & 15) == 0;
#define LM_ARGS                                                                                                      \
  grid, stream, (const bf16*)x, ld, oq, ok, ov, act, cos_t, sin_t, rd, key_scale, decay, state, q_start, slots, positions, \
      out, H, n, m, min_len, ws, maxseg, seg_len
#define LM_MODES(NT, V)                                                                                              \
  if (maxseg == 0) {                                                                                                 \
    lm_launch<NT, V, 0>(LM_ARGS);                                                                                    \
  } else {                                                                                                           \
    lm_launch<NT, V, 1>(LM_ARGS);                                                                                    \
    linear_attention_combine_kernel<<<dim3(nseq, H, (n * m + 255) / 256), 256, 0, stream>>>(                          \
        decay, state, q_start, slots, ws, H, n, m, min_len, maxseg, seg_len);                                        \
    if (maxseg > 1) lm_launch<NT, V, 2>(LM_ARGS);                                                                    \
  }
#define LM_RUN(NT)                 \
  if (vec) { LM_MODES(NT, true) }  \
  else { LM_MODES(NT, false) }
  if (n <= 32) { LM_RUN(1); }
  else if (n <= 64) { LM_RUN(2); }
  else if (n <= 96) { LM_RUN(3); }
  else { LM_RUN(4); }
#undef LM_RUN
#undef LM_MODES
#undef LM_ARGS
  GS_LAUNCH_CHECK("linear_attention_chunks");
  return 0;
}
