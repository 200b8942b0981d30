// H9 .. H12: feed-forward kernels. All math fp32; tensors bf16 (uint16_t storage) or fp32.
//
//   xielu            z = a + bias; z > 0: ap z^2 + z / 2; else an (e^z - 1 - z) + z / 2
//   silu_glu         gu = (gate | up) [T, 2F] -> silu(gate) * up
//   topk_softmax     per row of fp32 router logits: the `top` largest (lower index wins a tie) and
//                    the softmax over those alone
//   moe_rows         a few rows through their experts, two launches (the decode-step form of a
//                    mixture of gated experts, no host round trip so a graph can hold it):
//                    hid[t, k, :] = silu(Wg[e] h_t) * (Wu[e] h_t),  e = idx[t, k]
//                    out[t, :]    = sum_k wt[t, k] * Wd[e] hid[t, k, :]
//                    One wave per four output entries walks their weight rows in 16-byte loads (all
//                    in flight together) against the input row staged in LDS as fp32; a row's
//                    result does not depend on the others.
#include "../common.h"

namespace {

using rt::DT;

RT_DEVICE float sigm(float v) { return 1.0f / (1.0f + expf(-v)); }

template <typename T>
__global__ void __launch_bounds__(256) xielu_kernel(T* __restrict__ out, const T* __restrict__ a,
                                                    const float* __restrict__ bias, int64_t n, int F, float ap, float an) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float z = DT<T>::load(a + i) + (bias ? bias[i % F] : 0.f);
  DT<T>::store(out + i, z > 0.f ? ap * z * z + 0.5f * z : an * (expm1f(z) - z) + 0.5f * z);
}

template <typename T>
__global__ void __launch_bounds__(256) silu_glu_kernel(T* __restrict__ out, const T* __restrict__ gu, int64_t rows, int F) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * F) return;
  const int64_t r = i / F;
  const int c = (int)(i - r * F);
  const float g = DT<T>::load(gu + r * 2 * F + c);
  DT<T>::store(out + i, g * sigm(g) * DT<T>::load(gu + r * 2 * F + F + c));
}

constexpr int kTopPerLane = 8;      // experts per lane: up to 512 experts

// one wave: the `top` largest of a row of E logits (lower index wins a tie) and the softmax over them
RT_DEVICE void topk_row(int* __restrict__ idx, float* __restrict__ wt, const float* lg, int E, int top, int lane) {
  float v[kTopPerLane];
#pragma unroll
  for (int q = 0; q < kTopPerLane; ++q) {
    const int e = lane + 64 * q;
    v[q] = e < E ? lg[e] : -INFINITY;
  }
  float mine = 0.f, first = 0.f;      // lane k keeps the k-th chosen logit
  int mine_e = 0;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int be = 1 << 30;
#pragma unroll
    for (int q = 0; q < kTopPerLane; ++q)
      if (v[q] > best) {
        best = v[q];
        be = lane + 64 * q;
      }
    const float top_v = rt::wave_max(best);
    int cand = best == top_v ? be : 1 << 30;
    for (int o = 32; o; o >>= 1) cand = min(cand, __shfl_xor(cand, o));
#pragma unroll
    for (int q = 0; q < kTopPerLane; ++q)
      if (lane + 64 * q == cand) v[q] = -INFINITY;
    if (k == 0) first = top_v;
    if (lane == k) {
      mine = top_v;
      mine_e = min(cand, E - 1);     // (only all-NaN logits leave no candidate)
    }
  }
  const float e = lane < top ? expf(mine - first) : 0.f;
  const float sum = rt::wave_sum(e);
  if (lane < top) {
    idx[lane] = mine_e;
    wt[lane] = e / sum;
  }
}

__global__ void __launch_bounds__(64) topk_softmax_kernel(int* __restrict__ idx, float* __restrict__ wt,
                                                          const float* __restrict__ logits, int E, int top) {
  const int t = blockIdx.x;
  topk_row(idx + (size_t)t * top, wt + (size_t)t * top, logits + (size_t)t * E, E, top, threadIdx.x);
}

// router and choice in one launch: logits = W_router h (+ bias) in fp32 from the row in LDS — eight
// experts at a time, every lane's weight loads of a batch in flight together (16-byte loads when the
// row allows), wave sums, partials through LDS — then wave 0 chooses.
// dynamic LDS: the row [W], the logits [E], the partials [E][waves]
constexpr int kRouteBatch = 8;
template <typename T>
__global__ void __launch_bounds__(256) route_topk_kernel(int* __restrict__ idx, float* __restrict__ wt,
                                                         const T* __restrict__ h, const float* __restrict__ wr,
                                                         const float* __restrict__ bias, int W, int E, int top, int vec) {
  extern __shared__ float4 rl4[];       // (16-byte aligned: the row is read in 16-byte pieces)
  float* rl = reinterpret_cast<float*>(rl4);
  const int Wp = (W + 3) & ~3;
  float* lg = rl + Wp;
  float* part = lg + E;
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int c = threadIdx.x; c < W; c += blockDim.x) rl[c] = DT<T>::load(h + (size_t)t * W + c);
  __syncthreads();
  for (int e0 = 0; e0 < E; e0 += kRouteBatch) {
    float acc[kRouteBatch];
#pragma unroll
    for (int j = 0; j < kRouteBatch; ++j) acc[j] = 0.f;
    if (vec) {
      for (int c = threadIdx.x * 4; c < W; c += blockDim.x * 4) {
        const float4 x = *reinterpret_cast<const float4*>(rl + c);
        float4 w4[kRouteBatch];
#pragma unroll
        for (int j = 0; j < kRouteBatch; ++j)
          w4[j] = *reinterpret_cast<const float4*>(wr + (size_t)min(e0 + j, E - 1) * W + c);
#pragma unroll
        for (int j = 0; j < kRouteBatch; ++j) acc[j] += w4[j].x * x.x + w4[j].y * x.y + w4[j].z * x.z + w4[j].w * x.w;
      }
    } else {
      for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float x = rl[c];
#pragma unroll
        for (int j = 0; j < kRouteBatch; ++j) acc[j] += wr[(size_t)min(e0 + j, E - 1) * W + c] * x;
      }
    }
#pragma unroll
    for (int j = 0; j < kRouteBatch; ++j) {
      const float v = rt::wave_sum(acc[j]);
      if (lane == 0 && e0 + j < E) part[(e0 + j) * nw + wave] = v;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    float v = bias ? bias[e] : 0.f;
    for (int w = 0; w < nw; ++w) v += part[e * nw + w];
    lg[e] = v;
  }
  __syncthreads();
  if (wave == 0) topk_row(idx + (size_t)t * top, wt + (size_t)t * top, lg, E, top, lane);
}

// R dot products at once for the whole wave: rows w, w + rs, ... (the first `ok` of them) against
// x (fp32 in LDS), n entries each. The R rows' loads of a step are independent, so they are all in
// flight before the first multiply; x is read once per step for all rows.
template <int R>
RT_DEVICE void dot_rows_bf16(const uint16_t* __restrict__ w, size_t rs, int ok, const float* __restrict__ x, int n,
                             int lane, float* out) {
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  if ((n & 7) == 0 && (rs & 7) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
    for (int c = lane * 8; c < n; c += 512) {
      rt::short8 p[R];
#pragma unroll
      for (int r = 0; r < R; ++r) p[r] = *reinterpret_cast<const rt::short8*>(w + (size_t)(r < ok ? r : 0) * rs + c);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float xv = x[c + q];
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] += rt::bf2f((uint16_t)p[r][q]) * xv;
      }
    }
  } else {
    for (int c = lane; c < n; c += 64) {
      const float xv = x[c];
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] += rt::bf2f(w[(size_t)(r < ok ? r : 0) * rs + c]) * xv;
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) out[r] = rt::wave_sum(acc[r]);
}

template <int R>
RT_DEVICE void dot_rows_f32(const float* __restrict__ w, size_t rs, int ok, const float* __restrict__ x, int n, int lane,
                            float* out) {
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  if ((n & 3) == 0 && (rs & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
    for (int c = lane * 4; c < n; c += 256) {
      float4 p[R];
#pragma unroll
      for (int r = 0; r < R; ++r) p[r] = *reinterpret_cast<const float4*>(w + (size_t)(r < ok ? r : 0) * rs + c);
      const float x0 = x[c], x1 = x[c + 1], x2 = x[c + 2], x3 = x[c + 3];
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] += p[r].x * x0 + p[r].y * x1 + p[r].z * x2 + p[r].w * x3;
    }
  } else {
    for (int c = lane; c < n; c += 64) {
      const float xv = x[c];
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] += w[(size_t)(r < ok ? r : 0) * rs + c] * xv;
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) out[r] = rt::wave_sum(acc[r]);
}

template <int R>
RT_DEVICE void dot_rows(const uint16_t* w, size_t rs, int ok, const float* x, int n, int lane, float* out) {
  dot_rows_bf16<R>(w, rs, ok, x, n, lane, out);
}
template <int R>
RT_DEVICE void dot_rows(const float* w, size_t rs, int ok, const float* x, int n, int lane, float* out) {
  dot_rows_f32<R>(w, rs, ok, x, n, lane, out);
}

constexpr int kMoeWaves = 4;
constexpr int kMoeRows = 4;         // output entries a wave computes together
constexpr int kMoeBlock = kMoeWaves * kMoeRows;

// grid (T * top, blocks of kMoeBlock over F); wgu [E, 2F, W] = (gate | up) rows of every expert;
// act 1: experts without a gate, wgu [E, F, W], hidden = relu(up)^2
template <typename T>
__global__ void __launch_bounds__(64 * kMoeWaves) moe_gate_up_kernel(float* __restrict__ hid, const T* __restrict__ h,
                                                                     const T* __restrict__ wgu,
                                                                     const int* __restrict__ idx, int W, int F, int top,
                                                                     int act) {
  extern __shared__ float xs[];
  const int pair = blockIdx.x, t = pair / top;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = threadIdx.x; c < W; c += blockDim.x) xs[c] = DT<T>::load(h + (size_t)t * W + c);
  __syncthreads();
  const T* we = wgu + (size_t)idx[pair] * (act ? 1 : 2) * F * W;
  const int f = blockIdx.y * kMoeBlock + wave * kMoeRows;
  const int ok = min(kMoeRows, F - f);
  if (ok <= 0) return;
  float gv[kMoeRows], uv[kMoeRows];
  dot_rows<kMoeRows>(we + (size_t)f * W, (size_t)W, ok, xs, W, lane, gv);
  if (act) {
    if (lane < ok) {
      float u = 0.f;
#pragma unroll
      for (int r = 0; r < kMoeRows; ++r)
        if (r == lane) u = fmaxf(gv[r], 0.f);
      hid[(size_t)pair * F + f + lane] = u * u;
    }
    return;
  }
  dot_rows<kMoeRows>(we + (size_t)(F + f) * W, (size_t)W, ok, xs, W, lane, uv);
  if (lane < ok) {
    float g = 0.f, u = 0.f;
#pragma unroll
    for (int r = 0; r < kMoeRows; ++r)
      if (r == lane) {
        g = gv[r];
        u = uv[r];
      }
    hid[(size_t)pair * F + f + lane] = g * sigm(g) * u;
  }
}

// grid (T, blocks of kMoeBlock over W); wd [E, W, F]
template <typename T>
__global__ void __launch_bounds__(64 * kMoeWaves) moe_down_kernel(T* __restrict__ out, const float* __restrict__ hid,
                                                                  const T* __restrict__ wd, const int* __restrict__ idx,
                                                                  const float* __restrict__ wt, int W, int F, int top) {
  extern __shared__ float xs[];       // [top][F]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = threadIdx.x; c < top * F; c += blockDim.x) xs[c] = hid[(size_t)t * top * F + c];
  __syncthreads();
  const int c0 = blockIdx.y * kMoeBlock + wave * kMoeRows;
  const int ok = min(kMoeRows, W - c0);
  if (ok <= 0) return;
  float acc[kMoeRows];
#pragma unroll
  for (int r = 0; r < kMoeRows; ++r) acc[r] = 0.f;
  for (int k = 0; k < top; ++k) {
    float d[kMoeRows];
    dot_rows<kMoeRows>(wd + ((size_t)idx[(size_t)t * top + k] * W + c0) * F, (size_t)F, ok, xs + (size_t)k * F, F, lane, d);
    const float c = wt[(size_t)t * top + k];
#pragma unroll
    for (int r = 0; r < kMoeRows; ++r) acc[r] += c * d[r];
  }
  if (lane < ok) {
    float v = 0.f;
#pragma unroll
    for (int r = 0; r < kMoeRows; ++r)
      if (r == lane) v = acc[r];
    DT<T>::store(out + (size_t)t * W + c0 + lane, v);
  }
}

}  // namespace

void launch_xielu(void* out, const void* a, const float* bias, int64_t rows, int F, float ap, float an, bool bf,
                  hipStream_t stream) {
  const int64_t n = rows * F;
  if (n <= 0) return;
  const int blocks = (int)((n + 255) / 256);
  if (bf) xielu_kernel<uint16_t><<<blocks, 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)a, bias, n, F, ap, an);
  else xielu_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)a, bias, n, F, ap, an);
}

void launch_silu_glu(void* out, const void* gu, int64_t rows, int F, bool bf, hipStream_t stream) {
  const int64_t n = rows * F;
  if (n <= 0) return;
  const int blocks = (int)((n + 255) / 256);
  if (bf) silu_glu_kernel<uint16_t><<<blocks, 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)gu, rows, F);
  else silu_glu_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, rows, F);
}

int launch_topk_softmax(int* idx, float* wt, const float* logits, int T, int E, int top, hipStream_t stream) {
  if (T <= 0) return 0;
  if (E > 64 * kTopPerLane || top > 64 || top < 1 || top > E) return -1;
  topk_softmax_kernel<<<T, 64, 0, stream>>>(idx, wt, logits, E, top);
  return 0;
}

int launch_route_topk(int* idx, float* wt, const void* h, const float* wr, const float* bias, int T, int W, int E,
                      int top, bool bf, hipStream_t stream) {
  if (T <= 0) return 0;
  if (E > 64 * kTopPerLane || top > 64 || top < 1 || top > E) return -1;
  const size_t shm = sizeof(float) * ((size_t)((W + 3) & ~3) + 5 * (size_t)E);
  if (shm > 48 * 1024) return -2;
  const int vec = (W & 3) == 0 && (reinterpret_cast<uintptr_t>(wr) & 15) == 0 ? 1 : 0;
  if (bf) route_topk_kernel<uint16_t><<<T, 256, shm, stream>>>(idx, wt, (const uint16_t*)h, wr, bias, W, E, top, vec);
  else route_topk_kernel<float><<<T, 256, shm, stream>>>(idx, wt, (const float*)h, wr, bias, W, E, top, vec);
  return 0;
}

int launch_moe_rows(void* out, float* hid, const void* h, const void* wgu, const void* wd, const int* idx,
                    const float* wt, int T, int W, int F, int top, int act, bool bf, hipStream_t stream) {
  if (T <= 0) return 0;
  const size_t shm1 = sizeof(float) * (size_t)W, shm2 = sizeof(float) * (size_t)top * F;
  if (shm1 > 150 * 1024 || shm2 > 150 * 1024) return -1;
  // four output entries per wave: enough workgroups to fill the chip from a handful of rows
  const int pb = kMoeBlock;
  const dim3 g1(T * top, (F + pb - 1) / pb), g2(T, (W + pb - 1) / pb);
#define RT_MOE(TT)                                                                                                     \
  do {                                                                                                                 \
    auto k1 = moe_gate_up_kernel<TT>;                                                                                  \
    auto k2 = moe_down_kernel<TT>;                                                                                     \
    if (shm1 > 48 * 1024 &&                                                                                            \
        hipFuncSetAttribute((const void*)k1, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm1) != hipSuccess)     \
      return -2;                                                                                                       \
    if (shm2 > 48 * 1024 &&                                                                                            \
        hipFuncSetAttribute((const void*)k2, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm2) != hipSuccess)     \
      return -2;                                                                                                       \
    k1<<<g1, 64 * kMoeWaves, shm1, stream>>>(hid, (const TT*)h, (const TT*)wgu, idx, W, F, top, act);                    \
    k2<<<g2, 64 * kMoeWaves, shm2, stream>>>((TT*)out, hid, (const TT*)wd, idx, wt, W, F, top);                        \
  } while (0)
  if (bf) RT_MOE(uint16_t); else RT_MOE(float);
#undef RT_MOE
  return 0;
}
