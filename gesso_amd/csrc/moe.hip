// A mixture of small feed-forwards routed by a table over token ids: the token-by-token kernels.
//
// Token t with id v uses the experts table[v, 0 .. top-1], each with weight 1 / top; an expert is
// W_down act(W_up x), act(z) = relu(z)^2.  Expert weights lie stacked: up (E, F, H), down (E, H, F).
//
//   moe_table_up     a[t, k, :] = act(W_up[e_k] x_t)                       one block per (token, choice)
//   moe_table_down   y[t, :] = (1 / top) sum_k W_down[e_k] a[t, k, :]      one block per (token, 32 columns)
//                    (+ sigmoid(g_t) * s[t, :] when a shared expert's output s and its gate g are given)
//   relu_squared     act over the first F columns of rows (the shared expert's inner rows)
//
// A wavefront computes one output at a time: its lanes walk the weight row together (contiguous loads), each lane
// summing its columns in ascending order, then the lanes' sums are added in a fixed order; products and sums are
// float32.  Only the chosen experts' weights are read, which is what a step of few tokens needs; steps of many tokens
// go through the grouped products of moe_group.hip, which read an expert's weights once for all of its tokens.
#include "common.h"

template <typename T, typename TW>
__global__ void moe_table_up_kernel(const T* __restrict__ x, int ldx, const int* __restrict__ ids,
                                    const int* __restrict__ table, int top, const TW* __restrict__ up, int F, int H,
                                    T* __restrict__ a) {
  extern __shared__ float xs[];      // H floats
  const int t = blockIdx.x / top, k = blockIdx.x % top;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int j = threadIdx.x; j < H; j += blockDim.x) xs[j] = to_f32(x[(size_t)t * ldx + j]);
  __syncthreads();
  const int e = table[(size_t)ids[t] * top + k];
  const TW* w = up + (size_t)e * F * H;
  T* dst = a + ((size_t)t * top + k) * F;
  // rows of whole 16-byte pieces: eight weights a lane and load (the order of the sums depends on H alone)
  const bool vec = (H & 7) == 0 && aligned16(w);
  for (int f = blockIdx.y * nw + wave; f < F; f += gridDim.y * nw) {
    const TW* row = w + (size_t)f * H;
    float s = 0.f;
    if (vec) {
      for (int j = lane * 8; j < H; j += 512) {
        float w8[8];
        load8f(row + j, w8);
#pragma unroll
        for (int i = 0; i < 8; ++i) s = fmaf(w8[i], xs[j + i], s);
      }
    } else {
      for (int j = lane; j < H; j += 64) s = fmaf(to_f32(row[j]), xs[j], s);
    }
    s = wave_sum(s);
    if (lane == 0) {
      // the product is stored in the activation type before the activation, as a product of its own would be
      float z = to_f32(from_f32<T>(s));
      z = z > 0.f ? z : 0.f;
      dst[f] = from_f32<T>(z * z);
    }
  }
}

template <typename T, typename TW>
__global__ void moe_table_down_kernel(const T* __restrict__ a, const int* __restrict__ ids,
                                      const int* __restrict__ table, int top, const TW* __restrict__ down, int F, int H,
                                      const T* __restrict__ shared, const T* __restrict__ gate, int ldg,
                                      T* __restrict__ y) {
  extern __shared__ float as[];      // top * F floats
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int j = threadIdx.x; j < top * F; j += blockDim.x) as[j] = to_f32(a[(size_t)t * top * F + j]);
  __syncthreads();
  const float share = 1.0f / (float)top;
  float g = 0.f;
  if (shared) g = 1.f / (1.f + expf(-to_f32(gate[(size_t)t * ldg])));
  const bool vec = (F & 7) == 0 && aligned16(down);
  for (int i = blockIdx.y * nw + wave; i < H; i += gridDim.y * nw) {
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = table[(size_t)ids[t] * top + k];
      const TW* row = down + ((size_t)e * H + i) * F;
      float s = 0.f;
      if (vec) {
        for (int j = lane * 8; j < F; j += 512) {
          float w8[8];
          load8f(row + j, w8);
#pragma unroll
          for (int u = 0; u < 8; ++u) s = fmaf(w8[u], as[k * F + j + u], s);
        }
      } else {
        for (int j = lane; j < F; j += 64) s = fmaf(to_f32(row[j]), as[k * F + j], s);
      }
      total += wave_sum(s) * share;
    }
    if (lane == 0) {
      if (shared) total += g * to_f32(shared[(size_t)t * H + i]);
      y[(size_t)t * H + i] = from_f32<T>(total);
    }
  }
}

template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ x, int ldx, T* __restrict__ out, int F, long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long t = i / F;
  const int f = (int)(i % F);
  float z = to_f32(x[t * ldx + f]);
  z = z > 0.f ? z : 0.f;
  out[i] = from_f32<T>(z * z);
}

static int moe_blocks_y(int outputs, int tokens) {
  // enough blocks to fill the chip when tokens are few, one block a token when they are many
  int y = gs_ceil_div(outputs, 4);
  int cap = 2048 / (tokens > 0 ? tokens : 1);
  if (cap < 1) cap = 1;
  return y < cap ? y : cap;
}

extern "C" int gs_moe_table_up(const void* x, int dtype, int ldx, const int* ids, const int* table, int top,
                               const void* up, int w_dtype, int F, int H, void* a, int ntok, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && top > 0 && F > 0 && H > 0 && ldx >= H, "moe_table_up: bad sizes T=%d top=%d F=%d H=%d", ntok, top, F, H);
  GS_REQUIRE(H * sizeof(float) <= 65536, "moe_table_up: rows of %d are wider than the kernel's staging", H);
  if (ntok == 0) return 0;
  dim3 grid(ntok * top, moe_blocks_y(F, ntok * top));
  const size_t lds = H * sizeof(float);
  if (dtype == GS_F32 && w_dtype == GS_F32)
    moe_table_up_kernel<float, float><<<grid, 256, lds, stream>>>((const float*)x, ldx, ids, table, top, (const float*)up,
                                                                  F, H, (float*)a);
  else if (dtype == GS_BF16 && w_dtype == GS_BF16)
    moe_table_up_kernel<bf16, bf16><<<grid, 256, lds, stream>>>((const bf16*)x, ldx, ids, table, top, (const bf16*)up, F,
                                                                H, (bf16*)a);
  else if (dtype == GS_BF16 && w_dtype == GS_F32)
    moe_table_up_kernel<bf16, float><<<grid, 256, lds, stream>>>((const bf16*)x, ldx, ids, table, top, (const float*)up,
                                                                 F, H, (bf16*)a);
  else
    GS_REQUIRE(false, "moe_table_up: unsupported types %d %d", dtype, w_dtype);
  GS_LAUNCH_CHECK("moe_table_up");
  return 0;
}

extern "C" int gs_moe_table_down(const void* a, int dtype, const int* ids, const int* table, int top, const void* down,
                                 int w_dtype, int F, int H, const void* shared, const void* gate, int ldg, void* y,
                                 int ntok, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && top > 0 && F > 0 && H > 0, "moe_table_down: bad sizes T=%d top=%d F=%d H=%d", ntok, top, F, H);
  GS_REQUIRE((long)top * F * sizeof(float) <= 65536, "moe_table_down: %d x %d inner values are more than the kernel stages", top, F);
  GS_REQUIRE((shared == nullptr) == (gate == nullptr), "moe_table_down: a shared expert's rows come with their gate");
  if (ntok == 0) return 0;
  dim3 grid(ntok, moe_blocks_y(H, ntok));
  const size_t lds = (size_t)top * F * sizeof(float);
  if (dtype == GS_F32 && w_dtype == GS_F32)
    moe_table_down_kernel<float, float><<<grid, 256, lds, stream>>>((const float*)a, ids, table, top, (const float*)down,
                                                                    F, H, (const float*)shared, (const float*)gate, ldg,
                                                                    (float*)y);
  else if (dtype == GS_BF16 && w_dtype == GS_BF16)
    moe_table_down_kernel<bf16, bf16><<<grid, 256, lds, stream>>>((const bf16*)a, ids, table, top, (const bf16*)down, F,
                                                                  H, (const bf16*)shared, (const bf16*)gate, ldg,
                                                                  (bf16*)y);
  else if (dtype == GS_BF16 && w_dtype == GS_F32)
    moe_table_down_kernel<bf16, float><<<grid, 256, lds, stream>>>((const bf16*)a, ids, table, top, (const float*)down,
                                                                   F, H, (const bf16*)shared, (const bf16*)gate, ldg,
                                                                   (bf16*)y);
  else
    GS_REQUIRE(false, "moe_table_down: unsupported types %d %d", dtype, w_dtype);
  GS_LAUNCH_CHECK("moe_table_down");
  return 0;
}

extern "C" int gs_relu_squared(const void* x, int dtype, int ldx, void* out, int ntok, int F, hipStream_t stream) {
  GS_REQUIRE(ntok >= 0 && F > 0 && ldx >= F, "relu_squared: bad sizes T=%d F=%d ldx=%d", ntok, F, ldx);
  if (ntok == 0) return 0;
  const long total = (long)ntok * F;
  const int blocks = gs_ceil_div(total, 256);
  if (dtype == GS_F32)
    relu_squared_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, ldx, (float*)out, F, total);
  else if (dtype == GS_BF16)
    relu_squared_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)x, ldx, (bf16*)out, F, total);
  else
    GS_REQUIRE(false, "relu_squared: unknown dtype %d", dtype);
  GS_LAUNCH_CHECK("relu_squared");
  return 0;
}
