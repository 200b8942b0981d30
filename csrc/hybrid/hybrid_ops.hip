// H1, H2, H4 .. H7: the row-wise kernels of decoders that mix grouped attention with recurrent
// layers. All math fp32; tensors are bf16 (uint16_t storage) or fp32 as templated. One workgroup
// per row (H4: per sequence and 256 channels); rows are read twice (the second read hits L1 / L2),
// never staged in LDS, so any row width runs.
//
//   shift_norm        xs = x + y ; h = xs / rms(xs) * w ; out_m = h + (h_prev - h) * mu_m, m < n_mix
//                     h_prev: the row above inside a span, the sequence's state at a span's first
//                     row, zero at position 0; optionally stores h as the new state (decode step)
//                     (the norms of this file work on `groups` equal parts of a row, each divided
//                     by its own root mean square: blockIdx.y is the part)
//   shift_state       state[slot] = normed last row of every span
//   qk_prep           rotary pairs (2i, 2i + 1), per-head x / rms(x) (* a weight per channel; queries
//                     * 1 + coef ln(floor((p + 1) / every) + 1)); values optionally / rms(v);
//                     keys, values -> paged cache
//   mingru_scan       z = sigmoid(.), c = u + 1/2 | sigmoid(u); S = (1 - z) S + z c; out = S silu(g)
//   dual_norm_add     x += (a / rms(a) * wa + b / rms(b) * wb) / 2
//   add_norm          x += y ; out = x / rms(x) * w
//   limited_glu       g = min(gate, L), u = clamp(up, -L, L); g * sigmoid(1.702 g) * (u + 1)
#include "../common.h"

namespace {

using rt::DT;

RT_DEVICE float inv_rms(float ss, int n, float eps) { return 1.0f / sqrtf(ss / (float)n + eps); }
RT_DEVICE float sigmoidf(float v) { return 1.0f / (1.0f + expf(-v)); }
constexpr int kKeep = 4;    // entries per lane a two-pass row kernel keeps in registers (the rest are read again)

// block-wide sum of two values at once
RT_DEVICE void block_sum2(float& a, float& b, float* scratch) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  a = rt::wave_sum(a);
  b = rt::wave_sum(b);
  __syncthreads();
  if (lane == 0) {
    scratch[wid] = a;
    scratch[16 + wid] = b;
  }
  __syncthreads();
  a = rt::wave_sum(lane < nw ? scratch[lane] : 0.f);
  b = rt::wave_sum(lane < nw ? scratch[16 + lane] : 0.f);
}

template <typename OT, typename YT>
__global__ void __launch_bounds__(1024) shift_norm_kernel(
    OT* __restrict__ out, float* __restrict__ xs, const float* __restrict__ x, const YT* __restrict__ y,
    const float* __restrict__ w, const float* __restrict__ mu, float* __restrict__ state,
    const int* __restrict__ row_seq, const int64_t* __restrict__ positions, const int* __restrict__ start_pos,
    const int* __restrict__ slots, int W, int Wg, int n_mix, float eps, int store_state) {
  __shared__ float scratch[32];
  const int t = blockIdx.x;
  const int c0 = blockIdx.y * Wg;                        // this workgroup's part of the row
  const size_t T = gridDim.x;
  const int s = row_seq[t];
  const int64_t pos = positions[t];
  const bool first = pos == (int64_t)start_pos[s];      // first row of its span in this launch
  const float* xr = x + (size_t)t * W + c0;
  const YT* yr = y ? y + (size_t)t * W + c0 : nullptr;
  const float* xp = xr - W;                              // only read when !first (then t > 0)
  const YT* yp = yr ? yr - W : nullptr;
  float* st = state + (size_t)slots[s] * W + c0;
  const float* wg = w + c0;
  float ss = 0.f, sp = 0.f;
  float cv[kKeep], cu[kKeep];     // this row's and the row above's first entries per lane
  int i = 0;
  for (int c = threadIdx.x; c < Wg; c += blockDim.x, ++i) {
    const float v = xr[c] + (yr ? DT<YT>::load(yr + c) : 0.f);
    ss += v * v;
    float u = 0.f;
    if (!first) {
      u = xp[c] + (yp ? DT<YT>::load(yp + c) : 0.f);
      sp += u * u;
    }
#pragma unroll
    for (int j = 0; j < kKeep; ++j)
      if (j == i) {
        cv[j] = v;
        cu[j] = u;
      }
  }
  block_sum2(ss, sp, scratch);
  const float kc = inv_rms(ss, Wg, eps), kp = inv_rms(sp, Wg, eps);
  i = 0;
  for (int c = threadIdx.x; c < Wg; c += blockDim.x, ++i) {
    float v = 0.f, u = 0.f;
    if (i < kKeep) {
#pragma unroll
      for (int j = 0; j < kKeep; ++j)
        if (j == i) {
          v = cv[j];
          u = cu[j];
        }
    } else {
      v = xr[c] + (yr ? DT<YT>::load(yr + c) : 0.f);
      if (!first) u = xp[c] + (yp ? DT<YT>::load(yp + c) : 0.f);
    }
    const float h = v * kc * wg[c];
    float hp;
    if (!first) hp = u * kp * wg[c];
    else hp = pos > 0 ? st[c] : 0.f;
    for (int m = 0; m < n_mix; ++m)
      DT<OT>::store(out + ((size_t)m * T + t) * W + c0 + c, h + (hp - h) * mu[(size_t)m * W + c0 + c]);
    if (yr) xs[(size_t)t * W + c0 + c] = v;
    if (store_state) st[c] = h;
  }
}

__global__ void __launch_bounds__(1024) shift_state_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                           float* __restrict__ state, const int* __restrict__ cu_q,
                                                           const int* __restrict__ slots, int W, int Wg, float eps) {
  __shared__ float scratch[16];
  const int s = blockIdx.x;
  const int c0 = blockIdx.y * Wg;
  const int n = cu_q[s + 1] - cu_q[s];
  if (n <= 0) return;
  const float* xr = x + (size_t)(cu_q[s + 1] - 1) * W + c0;
  float ss = 0.f;
  for (int c = threadIdx.x; c < Wg; c += blockDim.x) ss += xr[c] * xr[c];
  const float k = inv_rms(rt::block_sum(ss, scratch), Wg, eps);
  float* st = state + (size_t)slots[s] * W + c0;
  for (int c = threadIdx.x; c < Wg; c += blockDim.x) st[c] = xr[c] * k * w[c0 + c];
}

// One wave per head unit: units 0 .. H - 1 are query heads, H .. H + G - 1 key heads (each also
// writes its value head). A lane holds entries lane, lane + 64, ... of the head (at most 4).
template <typename T>
__global__ void __launch_bounds__(1024) qk_prep_kernel(
    T* __restrict__ q, const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off, int v_from_k,
    const float* __restrict__ inv_freq, int rot_dims, float eps, const int64_t* __restrict__ positions,
    T* __restrict__ kc, T* __restrict__ vc, const int64_t* __restrict__ slot_mapping, int H, int G, int Dk, int Dv,
    int BS, int layout, const float* __restrict__ q_scale, const float* __restrict__ q_w,
    const float* __restrict__ k_w, int v_norm, float qt_coef, int qt_every) {
  __shared__ float cs_tab[256];      // (cos, sin) of the row's angles, once for all its heads
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < (rot_dims >> 1); i += blockDim.x) {
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    cs_tab[2 * i] = cs;
    cs_tab[2 * i + 1] = sn;
  }
  __syncthreads();
  const int64_t slot = slot_mapping[t];
  const int64_t blk = slot / BS;
  const int off = (int)(slot - blk * BS);
  const T* row = proj + (size_t)t * stride;
  for (int u = wave; u < H + G; u += nw) {
    const bool is_q = u < H;
    const T* src = row + (is_q ? q_off + u * Dk : k_off + (u - H) * Dk);
    float val[4];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = lane + 64 * j;
      float r = 0.f;
      if (d < Dk) {
        const float a = DT<T>::load(src + d);
        r = a;
        if (d < rot_dims) {
          const float b = DT<T>::load(src + (d ^ 1));
          const float cs = cs_tab[d & ~1], sn = cs_tab[d | 1];
          r = (d & 1) ? a * cs + b * sn : a * cs - b * sn;
        }
      }
      val[j] = r;
      ss += r * r;
    }
    float k = inv_rms(rt::wave_sum(ss), Dk, eps);
    if (is_q && q_scale) k *= q_scale[u];
    // the query factor grows with the logarithm of the position, in steps of qt_every positions
    if (is_q && qt_every > 0) k *= 1.0f + qt_coef * logf((float)((positions[t] + 1) / qt_every) + 1.0f);
    const float* cw = is_q ? q_w : k_w;                  // a learned weight per channel, or none
    // layout 1: the matrix-core attention kernels' cache (keys chunk-major per block, rt::kc_elem;
    // values transposed [Dv][BS])
    T* dst = is_q ? q + ((size_t)t * H + u) * Dk
                  : kc + ((size_t)blk * G + (u - H)) * BS * Dk + (layout ? 0 : (size_t)off * Dk);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = lane + 64 * j;
      if (d < Dk) DT<T>::store(dst + ((!is_q && layout) ? rt::kc_elem(BS, off, d) : d), val[j] * k * (cw ? cw[d] : 1.0f));
    }
    if (!is_q) {
      const int g = u - H;
      const T* vs = v_from_k ? src : row + v_off + g * Dv;
      T* vd = vc + ((size_t)blk * G + g) * BS * Dv;
      if (v_norm) {                                      // unit-RMS values, cached so
        float sv = 0.f;
        for (int d = lane; d < Dv; d += 64) {
          const float a = DT<T>::load(vs + d);
          sv += a * a;
        }
        const float kv = inv_rms(rt::wave_sum(sv), Dv, eps);
        for (int d = lane; d < Dv; d += 64)
          DT<T>::store(vd + (layout ? (size_t)d * BS + off : (size_t)off * Dv + d), DT<T>::load(vs + d) * kv);
      } else if (layout) for (int d = lane; d < Dv; d += 64) vd[(size_t)d * BS + off] = vs[d];
      else for (int d = lane; d < Dv; d += 64) vd[(size_t)off * Dv + d] = vs[d];
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256) mingru_scan_kernel(
    T* __restrict__ out, const T* __restrict__ proj, int stride, int z_off, int x_off, int g_off, int width,
    const float* __restrict__ bz, const float* __restrict__ bx, float* __restrict__ state,
    const int* __restrict__ cu_q, const int* __restrict__ start_pos, const int* __restrict__ slots) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int r0 = cu_q[s], r1 = cu_q[s + 1];
  if (c >= width || r1 <= r0) return;
  float* st = state + (size_t)slots[s] * width + c;
  float S = start_pos[s] > 0 ? *st : 0.f;
  const float bzc = bz[c], bxc = bx[c];
  for (int r = r0; r < r1; ++r) {
    const T* row = proj + (size_t)r * stride;
    const float z = sigmoidf(DT<T>::load(row + z_off + c) + bzc);
    const float u = DT<T>::load(row + x_off + c) + bxc;
    const float cand = u >= 0.f ? u + 0.5f : sigmoidf(u);
    const float g = DT<T>::load(row + g_off + c);
    S = (1.0f - z) * S + z * cand;
    DT<T>::store(out + (size_t)r * width + c, S * (g * sigmoidf(g)));
  }
  *st = S;
}

// The same recurrence for long spans, in three launches over chunks of kScanChunk rows: (1) every
// chunk alone from S = 0: its decay product A and its end state B; (2) per sequence, chunk by
// chunk: the state each chunk starts from (carry = A * carry + B), and the sequence's new state;
// (3) every chunk again from its true start state, writing the outputs. chunks [n, 2] = (sequence,
// first row), a sequence's chunks consecutive and in order; seq_chunk0 [S + 1] = first chunk of
// each sequence.
constexpr int kScanChunk = 64;

template <typename T, int PASS>
__global__ void __launch_bounds__(256) mingru_chunk_kernel(
    T* __restrict__ out, const T* __restrict__ proj, int stride, int z_off, int x_off, int g_off, int width,
    const float* __restrict__ bz, const float* __restrict__ bx, const int* __restrict__ cu_q,
    const int* __restrict__ chunks, float* __restrict__ ws_a, float* __restrict__ ws_b,
    const float* __restrict__ ws_in) {
  const int k = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int s = chunks[2 * k], r0 = chunks[2 * k + 1];
  const int r1 = min(r0 + kScanChunk, cu_q[s + 1]);
  const float bzc = bz[c], bxc = bx[c];
  float S = PASS == 1 ? 0.f : ws_in[(size_t)k * width + c];
  float A = 1.f;
  for (int r = r0; r < r1; ++r) {
    const T* row = proj + (size_t)r * stride;
    const float z = sigmoidf(DT<T>::load(row + z_off + c) + bzc);
    const float u = DT<T>::load(row + x_off + c) + bxc;
    const float cand = u >= 0.f ? u + 0.5f : sigmoidf(u);
    S = (1.0f - z) * S + z * cand;
    if (PASS == 1) {
      A *= 1.0f - z;
    } else {
      const float g = DT<T>::load(row + g_off + c);
      DT<T>::store(out + (size_t)r * width + c, S * (g * sigmoidf(g)));
    }
  }
  if (PASS == 1) {
    ws_a[(size_t)k * width + c] = A;
    ws_b[(size_t)k * width + c] = S;
  }
}

__global__ void __launch_bounds__(256) mingru_carry_kernel(const float* __restrict__ ws_a, const float* __restrict__ ws_b,
                                                           float* __restrict__ ws_in, float* __restrict__ state,
                                                           const int* __restrict__ seq_chunk0,
                                                           const int* __restrict__ start_pos,
                                                           const int* __restrict__ slots, int width) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int k0 = seq_chunk0[s], k1 = seq_chunk0[s + 1];
  if (c >= width || k1 <= k0) return;
  float* st = state + (size_t)slots[s] * width + c;
  float S = start_pos[s] > 0 ? *st : 0.f;
  for (int k = k0; k < k1; ++k) {
    ws_in[(size_t)k * width + c] = S;
    S = ws_a[(size_t)k * width + c] * S + ws_b[(size_t)k * width + c];
  }
  *st = S;
}

template <typename T>
__global__ void __launch_bounds__(1024) dual_norm_add_kernel(float* __restrict__ x, const T* __restrict__ a,
                                                             const float* __restrict__ wa, const T* __restrict__ b,
                                                             const float* __restrict__ wb, int W, float eps) {
  __shared__ float scratch[32];
  const T* ar = a + (size_t)blockIdx.x * W;
  const T* br = b + (size_t)blockIdx.x * W;
  float sa = 0.f, sb = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float u = DT<T>::load(ar + c), v = DT<T>::load(br + c);
    sa += u * u;
    sb += v * v;
  }
  block_sum2(sa, sb, scratch);
  const float ka = inv_rms(sa, W, eps), kb = inv_rms(sb, W, eps);
  float* xr = x + (size_t)blockIdx.x * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    xr[c] += 0.5f * (DT<T>::load(ar + c) * ka * wa[c] + DT<T>::load(br + c) * kb * wb[c]);
}

template <typename OT, typename YT>
__global__ void __launch_bounds__(1024) add_norm_kernel(OT* __restrict__ out, float* __restrict__ x,
                                                        const YT* __restrict__ y, const float* __restrict__ w, int W,
                                                        int Wg, float eps) {
  __shared__ float scratch[16];
  const int c0 = blockIdx.y * Wg;                        // this workgroup's part of the row
  float* xr = x + (size_t)blockIdx.x * W + c0;
  const YT* yr = y ? y + (size_t)blockIdx.x * W + c0 : nullptr;
  w += c0;
  out += (size_t)blockIdx.x * W + c0;
  float ss = 0.f;
  float cv[kKeep];
  int i = 0;
  for (int c = threadIdx.x; c < Wg; c += blockDim.x, ++i) {
    const float v = xr[c] + (yr ? DT<YT>::load(yr + c) : 0.f);
    ss += v * v;
#pragma unroll
    for (int j = 0; j < kKeep; ++j)
      if (j == i) cv[j] = v;
  }
  const float k = inv_rms(rt::block_sum(ss, scratch), Wg, eps);
  i = 0;
  for (int c = threadIdx.x; c < Wg; c += blockDim.x, ++i) {
    float v = 0.f;
    if (i < kKeep) {
#pragma unroll
      for (int j = 0; j < kKeep; ++j)
        if (j == i) v = cv[j];
    } else {
      v = xr[c] + (yr ? DT<YT>::load(yr + c) : 0.f);
    }
    if (yr) xr[c] = v;
    DT<OT>::store(out + c, v * k * w[c]);
  }
}

template <typename T>
__global__ void __launch_bounds__(256) limited_glu_kernel(T* __restrict__ out, const T* __restrict__ gu, int64_t rows,
                                                          int F, float limit) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * F) return;
  const int64_t r = i / F;
  const int c = (int)(i - r * F);
  const float g = fminf(DT<T>::load(gu + r * 2 * F + c), limit);
  const float u = fminf(fmaxf(DT<T>::load(gu + r * 2 * F + F + c), -limit), limit);
  DT<T>::store(out + i, g * sigmoidf(1.702f * g) * (u + 1.0f));
}

// bf16, F % 8 == 0: 16-byte loads and stores
__global__ void __launch_bounds__(256) limited_glu8_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ gu,
                                                           int64_t rows, int F, float limit) {
  const int F8 = F >> 3;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * F8) return;
  const int64_t r = i / F8;
  const int c = (int)(i - r * F8) * 8;
  const rt::short8 gv = *reinterpret_cast<const rt::short8*>(gu + r * 2 * F + c);
  const rt::short8 uv = *reinterpret_cast<const rt::short8*>(gu + r * 2 * F + F + c);
  rt::short8 o;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float g = fminf(rt::bf2f((uint16_t)gv[j]), limit);
    const float u = fminf(fmaxf(rt::bf2f((uint16_t)uv[j]), -limit), limit);
    o[j] = (short)rt::f2bf(g * sigmoidf(1.702f * g) * (u + 1.0f));
  }
  *reinterpret_cast<rt::short8*>(out + r * F + c) = o;
}

int row_threads(int W) {
  int t = 64;
  while (t < 1024 && t * 4 < W) t *= 2;
  return t;
}

}  // namespace

void launch_shift_norm(void* out, float* xs, const float* x, const void* y, const float* w, const float* mu,
                       float* state, const int* row_seq, const int64_t* positions, const int* start_pos,
                       const int* slots, int T, int W, int groups, int n_mix, float eps, bool out_bf, bool y_bf,
                       bool store_state, hipStream_t stream) {
  if (T <= 0) return;
  const int Wg = W / groups;
  const int th = row_threads(Wg);
  const dim3 grid(T, groups);
#define RT_SN(OT, YT)                                                                                                 \
  shift_norm_kernel<OT, YT><<<grid, th, 0, stream>>>((OT*)out, xs, x, (const YT*)y, w, mu, state, row_seq, positions, \
                                                     start_pos, slots, W, Wg, n_mix, eps, store_state ? 1 : 0)
  if (out_bf) {
    if (y_bf) RT_SN(uint16_t, uint16_t); else RT_SN(uint16_t, float);
  } else {
    if (y_bf) RT_SN(float, uint16_t); else RT_SN(float, float);
  }
#undef RT_SN
}

void launch_shift_state(const float* x, const float* w, float* state, const int* cu_q, const int* slots, int S, int W,
                        int groups, float eps, hipStream_t stream) {
  if (S <= 0) return;
  const int Wg = W / groups;
  shift_state_kernel<<<dim3(S, groups), row_threads(Wg), 0, stream>>>(x, w, state, cu_q, slots, W, Wg, eps);
}

void launch_qk_prep(void* q, const void* proj, int stride, int q_off, int k_off, int v_off, bool v_from_k,
                    const float* inv_freq, int rot_dims, float eps, const int64_t* positions, void* kc, void* vc,
                    const int64_t* slot_mapping, int T, int H, int G, int Dk, int Dv, int BS, bool bf, int layout,
                    const float* q_scale, const float* q_w, const float* k_w, bool v_norm, float qt_coef, int qt_every,
                    hipStream_t stream) {
  if (T <= 0) return;
  // one wave per head unit, up to 16 waves a row: a decode step's few rows spread over whole workgroups
  const int th = T > 64 ? 256 : 64 * (H + G < 4 ? 4 : H + G > 16 ? 16 : H + G);
  if (bf)
    qk_prep_kernel<uint16_t><<<T, th, 0, stream>>>((uint16_t*)q, (const uint16_t*)proj, stride, q_off, k_off, v_off,
                                                    v_from_k, inv_freq, rot_dims, eps, positions, (uint16_t*)kc,
                                                    (uint16_t*)vc, slot_mapping, H, G, Dk, Dv, BS, layout, q_scale,
                                                    q_w, k_w, v_norm ? 1 : 0, qt_coef, qt_every);
  else
    qk_prep_kernel<float><<<T, th, 0, stream>>>((float*)q, (const float*)proj, stride, q_off, k_off, v_off, v_from_k,
                                                 inv_freq, rot_dims, eps, positions, (float*)kc, (float*)vc,
                                                 slot_mapping, H, G, Dk, Dv, BS, layout, q_scale, q_w, k_w,
                                                 v_norm ? 1 : 0, qt_coef, qt_every);
}

void launch_mingru_scan(void* out, const void* proj, int stride, int z_off, int x_off, int g_off, int width,
                        const float* bz, const float* bx, float* state, const int* cu_q, const int* start_pos,
                        const int* slots, int S, bool bf, hipStream_t stream) {
  if (S <= 0 || width <= 0) return;
  const int th = width >= 256 ? 256 : 64;
  dim3 grid(S, (width + th - 1) / th);
  if (bf)
    mingru_scan_kernel<uint16_t><<<grid, th, 0, stream>>>((uint16_t*)out, (const uint16_t*)proj, stride, z_off, x_off,
                                                          g_off, width, bz, bx, state, cu_q, start_pos, slots);
  else
    mingru_scan_kernel<float><<<grid, th, 0, stream>>>((float*)out, (const float*)proj, stride, z_off, x_off, g_off,
                                                       width, bz, bx, state, cu_q, start_pos, slots);
}

int mingru_scan_chunk() { return kScanChunk; }

// ws: 3 * n_chunks * width floats
void launch_mingru_chunked(void* out, const void* proj, int stride, int z_off, int x_off, int g_off, int width,
                           const float* bz, const float* bx, float* state, const int* cu_q, const int* start_pos,
                           const int* slots, int S, const int* chunks, int n_chunks, const int* seq_chunk0, float* ws,
                           bool bf, hipStream_t stream) {
  if (S <= 0 || width <= 0 || n_chunks <= 0) return;
  const int th = width >= 256 ? 256 : 64;
  const int cb = (width + th - 1) / th;
  float *wa = ws, *wb = ws + (size_t)n_chunks * width, *wi = ws + 2 * (size_t)n_chunks * width;
  dim3 gc(n_chunks, cb), gs(S, cb);
#define RT_MG(TT)                                                                                                      \
  do {                                                                                                                 \
    mingru_chunk_kernel<TT, 1><<<gc, th, 0, stream>>>((TT*)out, (const TT*)proj, stride, z_off, x_off, g_off, width,  \
                                                      bz, bx, cu_q, chunks, wa, wb, nullptr);                         \
    mingru_carry_kernel<<<gs, th, 0, stream>>>(wa, wb, wi, state, seq_chunk0, start_pos, slots, width);               \
    mingru_chunk_kernel<TT, 3><<<gc, th, 0, stream>>>((TT*)out, (const TT*)proj, stride, z_off, x_off, g_off, width,  \
                                                      bz, bx, cu_q, chunks, nullptr, nullptr, wi);                    \
  } while (0)
  if (bf) RT_MG(uint16_t); else RT_MG(float);
#undef RT_MG
}

void launch_dual_norm_add(float* x, const void* a, const float* wa, const void* b, const float* wb, int T, int W,
                          float eps, bool bf, hipStream_t stream) {
  if (T <= 0) return;
  if (bf)
    dual_norm_add_kernel<uint16_t><<<T, row_threads(W), 0, stream>>>(x, (const uint16_t*)a, wa, (const uint16_t*)b, wb,
                                                                     W, eps);
  else
    dual_norm_add_kernel<float><<<T, row_threads(W), 0, stream>>>(x, (const float*)a, wa, (const float*)b, wb, W, eps);
}

void launch_add_norm(void* out, float* x, const void* y, const float* w, int T, int W, int groups, float eps,
                     bool out_bf, bool y_bf, hipStream_t stream) {
  if (T <= 0) return;
  const int Wg = W / groups;
  const int th = row_threads(Wg);
  const dim3 grid(T, groups);
#define RT_AN(OT, YT) add_norm_kernel<OT, YT><<<grid, th, 0, stream>>>((OT*)out, x, (const YT*)y, w, W, Wg, eps)
  if (out_bf) {
    if (y_bf) RT_AN(uint16_t, uint16_t); else RT_AN(uint16_t, float);
  } else {
    if (y_bf) RT_AN(float, uint16_t); else RT_AN(float, float);
  }
#undef RT_AN
}

void launch_limited_glu(void* out, const void* gu, int64_t rows, int F, float limit, bool bf, hipStream_t stream) {
  const int64_t n = rows * F;
  if (n <= 0) return;
  if (bf && F % 8 == 0) {
    limited_glu8_kernel<<<(int)((n / 8 + 255) / 256), 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)gu, rows, F, limit);
    return;
  }
  const int blocks = (int)((n + 255) / 256);
  if (bf) limited_glu_kernel<uint16_t><<<blocks, 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)gu, rows, F, limit);
  else limited_glu_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, rows, F, limit);
}
