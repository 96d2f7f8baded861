// Attention over cached latent rows on the matrix cores (bfloat16 storage): prompt portions and single tokens alike.
//
// Every head of a token attends over the same rows [z | k_rot] (D = c + r columns; the first c are also the values),
// so what a block shares through LDS is one tile of rows for all of its queries: a block owns up to 64 query rows
// (token, head) of one sequence, consecutive tokens x up to 64 heads, 16 rows a wavefront; a step stages KSTEP cached
// rows once, row-major for the score product and transposed (column-major) for the value product.
//
// Both products are computed transposed (v_mfma_f32_16x16x32_bf16), so that all a lane holds concerns one query row
// (lane % 16) and no softmax weight crosses lanes:
//   S^T = R Q^T     A = staged rows (lane l: row l % 16 of a block of 16, columns 8 (l / 16) .. + 7 of a step of 32),
//                   B = the wavefront's query fragments (registers); lane l gets rows 4 (l / 16) + 0..3 of the block.
//   O^T = Z^T P^T   B = the lane's own eight weights of a chunk of 32 rows (two blocks of four), A = the transposed
//                   values read in the same order; lane l gets value columns 4 (l / 16) + 0..3 of a tile of 16.
// Scores, maxima, sums and softmax weights are float32.  A weight enters the matrix cores as the sum of two bfloat16
// numbers (its rounding and the rounding of what that left over), two products a chunk: the weights keep 16 bits
// of mantissa, and the sums are float32.
//
// The query at position p sees rows lo..p of its sequence, lo = 0 or p - window + 1; a block walks from the oldest row
// any of its queries sees to its last query's own, each row masked per query.  Rows past the block's last are staged
// as zeros (their pages may belong to nobody).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;

#define LM_LOG2E 1.4426950408889634f
#define LM_ROWS 64     // query rows a block

// CT: the most tiles of 16 value columns (c <= 16 CT); the score product takes up to CT / 2 + 2 steps of 32 columns.
template <int CT, int KSTEP>
__global__ __launch_bounds__(256) void attention_latent_mfma_kernel(
    const bf16* __restrict__ qa, const bf16* __restrict__ cache, const int* __restrict__ positions,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_row, const int* __restrict__ tile_n,
    const int* __restrict__ block_table, int max_blocks, int page_size, int window, float scale,
    bf16* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int nsplit, int rows_total, int H,
    int HB, int c, int D) {
  constexpr int DK = CT / 2 + 2;
  constexpr int NB = KSTEP / 16, NC = KSTEP / 32, VROW = KSTEP + 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int Dp = (D + 31) & ~31, krow = Dp + 8;
  bf16* ks = reinterpret_cast<bf16*>(lds);                                            // [KSTEP][krow]
  uint16_t* vt = reinterpret_cast<uint16_t*>(lds + (size_t)KSTEP * krow * 2);         // [c up to whole 64][VROW]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r16 = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x;
  int seq = tile, row0 = tile, nt = 1;               // without a list: sequence i brings the single token i
  if (tile_seq) {
    seq = tile_seq[tile];
    row0 = tile_row[tile];
    nt = tile_n[tile];
  }
  const int h0 = blockIdx.y * HB;
  const int hb = H - h0 < HB ? H - h0 : HB;
  const int nrows = nt * hb;
  const int pos0 = positions[row0];                  // a tile's tokens stand at consecutive positions
  const int* bt = block_table + (size_t)seq * max_blocks;
  // A block with at most 16 query rows (a single token of up to 16 heads): every wavefront holds the same rows and
  // computes the same scores, and takes a quarter of the value columns.
  const bool share = nrows <= 16;
  const int wrow = share ? 0 : wave * 16;
  const int m = wrow + r16;
  const bool valid = m < nrows;
  const int ti = valid ? m / hb : 0, head = h0 + (valid ? m % hb : 0);
  const int pos = pos0 + ti;
  const size_t qrow = (size_t)(row0 + ti) * H + head;
  const bool wave_on = wrow < nrows;
  const int ti_lo = wrow / hb;
  const int ti_hi = (wrow + 15) / hb < nt - 1 ? (wrow + 15) / hb : nt - 1;

  bf16x8_t qf[DK];
#pragma unroll
  for (int kk = 0; kk < DK; ++kk) {
    const int f = 32 * kk + 8 * g;
    u32x4_t v = {0u, 0u, 0u, 0u};
    if (valid && f < D) v = *reinterpret_cast<const u32x4_t*>(qa + qrow * D + f);
    qf[kk] = __builtin_bit_cast(bf16x8_t, v);
  }
  f32x4_t acc[CT];
#pragma unroll
  for (int dt = 0; dt < CT; ++dt) acc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float mrun = -INFINITY, lrun = 0.f;
  const float sc = scale * LM_LOG2E;
  const int kmax = pos0 + nt - 1;
  const int kmin = window > 0 ? (pos0 - window + 1 > 0 ? pos0 - window + 1 : 0) : 0;
  const int chunks = Dp >> 3, ct = c >> 4;
  // value tiles go in groups of four (a last group may reach past c: its spare tiles are computed on LDS rows that
  // belong to nobody and never stored); with shared rows a wavefront takes a quarter of the groups
  const int ngr = (ct + 3) >> 2, gq = (ngr + 3) >> 2;
  const int g_lo = share ? wave * gq : 0;
  const int g_hi = share ? ((wave + 1) * gq < ngr ? (wave + 1) * gq : ngr) : ngr;
  const int dt_lo = 4 * g_lo, dt_hi = 4 * g_hi < ct ? 4 * g_hi : ct;
  // with the rows shared out over nsplit blocks (blockIdx.z), each takes a run of whole steps
  const int nsteps = (kmax - kmin) / KSTEP + 1;
  const int per = (nsteps + nsplit - 1) / nsplit;
  const int s_begin = kmin + (int)blockIdx.z * per * KSTEP;
  const int s_last = kmin + ((int)blockIdx.z + 1) * per * KSTEP - 1 < kmax ? kmin + ((int)blockIdx.z + 1) * per * KSTEP - 1 : kmax;

  // This thread's pieces of a step's rows: 16 bytes each.  A step's pieces are asked for while the step before it is
  // computed, all of them before any is waited for, and go into LDS after that step's products: row-major for the
  // scores, and their value columns transposed.  Of a wavefront's 64 pieces sixteen rows have four neighbouring pieces
  // each: 64 contiguous bytes a row from memory, and the transposed 2-byte stores of one instruction fall into
  // different LDS banks (sixteen neighbouring rows of one column are eight words; the four column groups lie 16 banks
  // apart).
  // All pieces of a thread belong to one row of the step (its pieces lie whole wavefronts of four apart, and the rows
  // repeat every KSTEP / 16 wavefronts), so a step costs a thread one page lookup; where a piece goes in LDS is the
  // same in every step.
  constexpr int NL = KSTEP * (DK * 4) / 256;
  const int pk = ((tid >> 6) % (KSTEP / 16)) * 16 + (lane & 15);       // this thread's row of a step
  int pf[NL];                                                         // its pieces' columns (< 0: none)
  bf16* ksp[NL];
  uint16_t* vtp[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int unit = (tid >> 6) + 4 * i;
    const int ch = (unit / (KSTEP / 16)) * 4 + (lane >> 4);
    pf[i] = ch < chunks ? ch * 8 : -1;
    ksp[i] = ks + (size_t)pk * krow + ch * 8;
    vtp[i] = vt + (size_t)ch * 8 * VROW + pk;
  }
  u32x4_t pv[NL];
#define LM_ASK(s0)                                                                                              \
  {                                                                                                             \
    const int j = (s0) + pk;                                                                                    \
    const bool row_in = j <= kmax;                                                                              \
    const int jj = row_in ? j : kmax;                                                                           \
    const bf16* src = cache + ((size_t)bt[jj / page_size] * page_size + jj % page_size) * D;                    \
    _Pragma("unroll") for (int i = 0; i < NL; ++i) {                                                            \
      pv[i] = u32x4_t{0u, 0u, 0u, 0u};                                                                          \
      if (row_in && pf[i] >= 0 && pf[i] < D) pv[i] = *reinterpret_cast<const u32x4_t*>(src + pf[i]);            \
    }                                                                                                           \
  }
  if (s_begin <= s_last) LM_ASK(s_begin);
  for (int s0 = s_begin; s0 <= s_last; s0 += KSTEP) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NL; ++i)
      if (pf[i] >= 0) {
        *reinterpret_cast<u32x4_t*>(ksp[i]) = pv[i];
        if (pf[i] < c) {
          const unsigned w[4] = {pv[i].x, pv[i].y, pv[i].z, pv[i].w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            vtp[i][(2 * e) * VROW] = (uint16_t)(w[e] & 0xffffu);
            vtp[i][(2 * e + 1) * VROW] = (uint16_t)(w[e] >> 16);
          }
        }
      }
    __syncthreads();
    if (s0 + KSTEP <= s_last) LM_ASK(s0 + KSTEP);
    // a wavefront none of whose queries sees a row of this step waits for the next
    const bool step_on = wave_on && s0 <= pos0 + ti_hi && (window <= 0 || s0 + KSTEP - 1 > pos0 + ti_lo - window);
    if (!step_on) continue;
    // (products that follow each other in the code belong to different accumulators: one that waits for the result of
    // the one before it would leave the matrix cores idle for its whole latency)
    f32x4_t st[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) st[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < DK; ++kk)
      if (32 * kk < D) {
        bf16x8_t a[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b)
          a[b] = *reinterpret_cast<const bf16x8_t*>(ks + (size_t)(16 * b + r16) * krow + 32 * kk + 8 * g);
#pragma unroll
        for (int b = 0; b < NB; ++b) st[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b], qf[kk], st[b], 0, 0, 0);
      }
    float mstep = -INFINITY;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int j = s0 + 16 * b + 4 * g + e;
        const bool seen = valid && j <= pos && (window <= 0 || j > pos - window);
        const float s = seen ? st[b][e] * sc : -INFINITY;
        st[b][e] = s;
        mstep = fmaxf(mstep, s);
      }
    mstep = group4_max(mstep);
    const float mnew = fmaxf(mrun, mstep);
    const float muse = mnew == -INFINITY ? 0.f : mnew;         // a query that has seen nothing yet
    const float alpha = __builtin_amdgcn_exp2f(mrun - muse);
    float psum = 0.f;
    bf16x8_t phi[NC], plo[NC];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float p = __builtin_amdgcn_exp2f(st[b][e] - muse);
        psum += p;
        const __bf16 hi = (__bf16)p;
        phi[b >> 1][(b & 1) * 4 + e] = hi;
        plo[b >> 1][(b & 1) * 4 + e] = (__bf16)(p - (float)hi);
      }
    psum = group4_sum(psum);
    lrun = lrun * alpha + psum;
    mrun = mnew;
    // value columns in groups of four tiles: eight independent products side by side (four tiles, each with the
    // weights' first and second term)
#pragma unroll
    for (int g4 = 0; g4 < CT / 4; ++g4)
      if (g4 >= g_lo && g4 < g_hi) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[4 * g4 + u][e] *= alpha;
#pragma unroll
        for (int ch = 0; ch < NC; ++ch) {
          bf16x8_t a[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const uint16_t* vr = vt + (size_t)(16 * (4 * g4 + u) + r16) * VROW + 32 * ch + 4 * g;
            const u32x2_t v0 = *reinterpret_cast<const u32x2_t*>(vr);
            const u32x2_t v1 = *reinterpret_cast<const u32x2_t*>(vr + 16);
            a[u] = __builtin_bit_cast(bf16x8_t, (u32x4_t{v0.x, v0.y, v1.x, v1.y}));
          }
#pragma unroll
          for (int u = 0; u < 4; ++u)
            acc[4 * g4 + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], phi[ch], acc[4 * g4 + u], 0, 0, 0);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            acc[4 * g4 + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], plo[ch], acc[4 * g4 + u], 0, 0, 0);
        }
      }
  }
  if (!valid) return;
  if (nsplit > 1) {
    // this block's share: the running maximum (base 2), the sum, and the weighted values not yet divided
    const size_t prow = (size_t)blockIdx.z * rows_total + qrow;
    if (g == 0 && (!share || wave == 0)) {
      part_ml[prow * 2] = mrun;
      part_ml[prow * 2 + 1] = lrun;
    }
#pragma unroll
    for (int dt = 0; dt < CT; ++dt)
      if (dt >= dt_lo && dt < dt_hi)
        *reinterpret_cast<f32x4_t*>(part_o + prow * c + 16 * dt + 4 * g) = acc[dt];
    return;
  }
  const float inv = 1.0f / lrun;
#pragma unroll
  for (int dt = 0; dt < CT; ++dt)
    if (dt >= dt_lo && dt < dt_hi) {
      u32x2_t w;
      w.x = (unsigned)f32_to_bf16(acc[dt][0] * inv).x | ((unsigned)f32_to_bf16(acc[dt][1] * inv).x << 16);
      w.y = (unsigned)f32_to_bf16(acc[dt][2] * inv).x | ((unsigned)f32_to_bf16(acc[dt][3] * inv).x << 16);
      *reinterpret_cast<u32x2_t*>(out + qrow * c + 16 * dt + 4 * g) = w;
    }
}

// out[row, :] = sum_z part_o[z, row, :] 2^(m_z - M) / sum_z l_z 2^(m_z - M), M = max_z m_z: the shares of the blocks
// that walked a row's keys in parts, added in the order of the parts.
__global__ void attention_latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                              int nsplit, int rows_total, int c, bf16* __restrict__ out) {
  __shared__ float wz[64];           // the parts' weights 2^(m_z - M) / L (at most 64 parts)
  const int row = blockIdx.x, lane = threadIdx.x & 63;
  // every wavefront of the block finds the weights itself: lane z holds part z
  float m = -INFINITY, l = 0.f;
  if (lane < nsplit) {
    const float* ml = part_ml + ((size_t)lane * rows_total + row) * 2;
    m = ml[0];
    l = ml[1];
  }
  const float M = wave_max(m);
  const float w = lane < nsplit ? __builtin_amdgcn_exp2f(m - M) : 0.f;
  const float L = wave_sum(l * w);
  if (threadIdx.x < 64) wz[lane] = w / L;
  __syncthreads();
  for (int j = threadIdx.x; j < c; j += blockDim.x) {
    float a = 0.f;
    for (int z = 0; z < nsplit; ++z) a += part_o[((size_t)z * rows_total + row) * c + j] * wz[z];
    out[(size_t)row * c + j] = f32_to_bf16(a);
  }
}

// Whether the kernel takes these sizes: value columns in whole tiles of 16 up to 512, rows of whole 16-byte pieces,
// rotated columns that fit the score product's steps.
extern "C" int gs_attention_latent_mfma_supports(int H, int c, int r) {
  const int D = c + r;
  if (H <= 0 || c <= 0 || r < 0 || c % 16 || D % 8) return 0;
  if (c <= 128 && D <= 32 * (8 / 2 + 2)) return 1;
  if (c <= 512 && D <= 32 * (32 / 2 + 2)) return 1;
  return 0;
}

// How many consecutive tokens of a sequence one block takes (the host cuts its tile list by this).
extern "C" int gs_attention_latent_mfma_tokens(int H) {
  const int hb = H < LM_ROWS ? H : LM_ROWS;
  return LM_ROWS / hb;
}

extern "C" int gs_attention_latent_mfma(const void* qa, const void* cache, const int* positions, const int* tile_seq,
                                        const int* tile_row, const int* tile_n, int ntiles, const int* block_table,
                                        int max_blocks, int page_size, int window, float scale, void* out, int H, int c,
                                        int r, int nsplit, float* part_o, float* part_ml, int ntok, hipStream_t stream) {
  GS_REQUIRE(gs_attention_latent_mfma_supports(H, c, r), "attention_latent_mfma: sizes H=%d c=%d r=%d are not taken", H, c, r);
  GS_REQUIRE(ntiles >= 0 && page_size > 0 && max_blocks > 0 && window >= 0, "attention_latent_mfma: bad tiles/page_size/max_blocks/window");
  GS_REQUIRE((tile_seq == nullptr) == (tile_row == nullptr) && (tile_seq == nullptr) == (tile_n == nullptr),
             "attention_latent_mfma: a tile list has three rows");
  GS_REQUIRE(nsplit >= 1 && nsplit <= 64 && (nsplit == 1 || (part_o && part_ml)), "attention_latent_mfma: %d parts need their room", nsplit);
  if (ntiles == 0) return 0;
  const int D = c + r, Dp = (D + 31) & ~31;
  const int rows_total = ntok * H;
  const int HB = H < LM_ROWS ? H : LM_ROWS;
  const int hgroups = gs_ceil_div(H, HB);
  GS_REQUIRE(hgroups <= 65535, "attention_latent_mfma: too many heads");
  dim3 grid(ntiles, hgroups, nsplit);
  if (c <= 128 && D <= 32 * (8 / 2 + 2)) {
    const size_t lds = (size_t)64 * (Dp + 8) * 2 + (size_t)((c + 63) & ~63) * (64 + 4) * 2;
    attention_latent_mfma_kernel<8, 64><<<grid, 256, lds, stream>>>(
        (const bf16*)qa, (const bf16*)cache, positions, tile_seq, tile_row, tile_n, block_table, max_blocks, page_size,
        window, scale, (bf16*)out, part_o, part_ml, nsplit, rows_total, H, HB, c, D);
  } else if (c <= 256 && D <= 32 * (16 / 2 + 2)) {
    // latents up to 256: half the accumulators of the widest form, so steps of 64 rows fit
    const size_t lds = (size_t)64 * (Dp + 8) * 2 + (size_t)((c + 63) & ~63) * (64 + 4) * 2;
    static bool raised_mid = false;
    if (!raised_mid) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_latent_mfma_kernel<16, 64>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
      GS_REQUIRE(e == hipSuccess, "attention_latent_mfma: cannot raise the LDS limit: %s", hipGetErrorString(e));
      raised_mid = true;
    }
    GS_REQUIRE(lds <= 96 * 1024, "attention_latent_mfma: %zu bytes of LDS", lds);
    attention_latent_mfma_kernel<16, 64><<<grid, 256, lds, stream>>>(
        (const bf16*)qa, (const bf16*)cache, positions, tile_seq, tile_row, tile_n, block_table, max_blocks, page_size,
        window, scale, (bf16*)out, part_o, part_ml, nsplit, rows_total, H, HB, c, D);
  } else {
    const size_t lds = (size_t)32 * (Dp + 8) * 2 + (size_t)((c + 63) & ~63) * (32 + 4) * 2;
    static bool raised = false;
    if (!raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_latent_mfma_kernel<32, 32>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
      GS_REQUIRE(e == hipSuccess, "attention_latent_mfma: cannot raise the LDS limit: %s", hipGetErrorString(e));
      raised = true;
    }
    GS_REQUIRE(lds <= 96 * 1024, "attention_latent_mfma: %zu bytes of LDS", lds);
    attention_latent_mfma_kernel<32, 32><<<grid, 256, lds, stream>>>(
        (const bf16*)qa, (const bf16*)cache, positions, tile_seq, tile_row, tile_n, block_table, max_blocks, page_size,
        window, scale, (bf16*)out, part_o, part_ml, nsplit, rows_total, H, HB, c, D);
  }
  GS_LAUNCH_CHECK("attention_latent_mfma");
  if (nsplit > 1) {
    attention_latent_merge_kernel<<<rows_total, c >= 256 ? 256 : 64, 0, stream>>>(part_o, part_ml, nsplit, rows_total, c, (bf16*)out);
    GS_LAUNCH_CHECK("attention_latent_merge");
  }
  return 0;
}
