// C1 - C4, C6 - C8: the row-wise kernels around input convolutions, whole-projection norms and
// matrix-state recurrences. All math fp32; activations are bf16 (uint16_t storage) or fp32 as
// templated; the residual stream, the convolution states and everything that enters a recurrence
// are fp32. One workgroup per row (256 lanes), rows are re-read from L1 / L2, so any width runs.
//
//   canon_add        xs = x + (y + y2) / rms(y + y2) * nw ; h_t = xs_t + sum_k cw[:, taps-1-k] xs_(t-k)
//                    rows ahead of a span come from the sequence's state slot, zeros ahead of position 0
//   conv_state       shift a sequence's convolution state by its rows of this batch
//   qkv_prep_wide    biases, RMS norm over the whole query / key row with a weight per channel,
//                    rotation in halves (cos / sin times a magnitude), values turned by their
//                    position or taken from the biased keys; keys / values -> the paged cache
//   turn_back        attention output turned in halves by minus the position, scaled
//   silu_cols        fp32 silu of a column range
//   removal_prep     r, k, v, decay, removal rate * unit key, unit key of a generalized delta rule
//   delta_prep       short convolutions + silu, unit q / k, step size and decay of a gated delta rule
//   head_norm_gate   per-head or whole-row RMS norm, weight, sigmoid / silu gate, scale
//   relu2            relu(a)^2
#include "../common.h"

namespace {

using rt::DT;
constexpr int kMaxTaps = 16;
constexpr int kThreads = 256;

RT_DEVICE float sigm(float x) { return 1.0f / (1.0f + __expf(-x)); }
RT_DEVICE float silu(float x) { return x * sigm(x); }

// tap k of row t reads k tokens back: kind 1 = row t - k of this batch, 2 = the state, 0 = zeros
struct Tap {
  int kind;
  size_t at;      // kind 1: row index; kind 2: state row
};
RT_DEVICE Tap tap_of(int k, int t, int local, int64_t pos, int taps) {
  Tap r;
  r.kind = 0;
  r.at = 0;
  if (local >= k) {
    r.kind = 1;
    r.at = (size_t)(t - k);
  } else if (pos >= k) {
    r.kind = 2;
    r.at = (size_t)(taps - 1 - k + local);
  }
  return r;
}

// state layout: state[slot][sub][i][W], i < keep (= max(taps - 1, 1) rows), oldest first: row i of a
// sequence whose span starts at position p0 holds the input of position p0 - (taps - 1) + i.
// TAPS: the taps as a compile-time number (0: no convolution, only the add), or kMaxTaps for any
// number up to that (`taps` at run time)
template <typename OT, typename YT, int TAPS>
__global__ void __launch_bounds__(1024) canon_add_kernel(
    OT* __restrict__ h, float* __restrict__ xs, const float* __restrict__ x, const YT* __restrict__ y,
    const YT* __restrict__ y2, const float* __restrict__ nw, float eps, const float* __restrict__ cw,
    float* __restrict__ state, int sub, int nsub, const int* __restrict__ row_seq, const int64_t* __restrict__ positions,
    const int* __restrict__ start_pos, const int* __restrict__ slots, int W, int taps, int keep, int shift_state) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  // (loops over the taps are unrolled with a guard, so that per-tap values stay in registers)
  constexpr int NT = TAPS == 0 ? 1 : TAPS;
  if (TAPS != kMaxTaps) taps = TAPS;
  float inv[NT];
  float* st = nullptr;
  int64_t pos = 0;
  int local = 0;
  if (cw != nullptr) {
    const int s = row_seq[t];
    pos = positions[t];
    local = (int)(pos - start_pos[s]);
    st = state + ((size_t)slots[s] * nsub + sub) * keep * W;
  } else {
    taps = 1;     // only the add: tap 0 is this row
  }
#pragma unroll
  for (int k = 0; k < NT; ++k) {
    inv[k] = 0.f;
    if (k < taps && y != nullptr) {
      const Tap tp = tap_of(k, t, local, pos, taps);
      if (tp.kind == 1) {
        const YT* yr = y + tp.at * W;
        const YT* y2r = y2 ? y2 + tp.at * W : nullptr;
        float ss = 0.f;
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
          const float v = DT<YT>::load(yr + c) + (y2r ? DT<YT>::load(y2r + c) : 0.f);
          ss += v * v;
        }
        inv[k] = rsqrtf(rt::block_sum(ss, scratch) / W + eps);
      }
    }
  }
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float acc = 0.f, v0 = 0.f;
    const float nwc = y != nullptr ? nw[c] : 0.f;
#pragma unroll
    for (int k = 0; k < NT; ++k) {
      if (k < taps) {
        const Tap tp = tap_of(k, t, local, pos, taps);
        float v = 0.f;
        if (tp.kind == 1) {
          v = x[tp.at * W + c];
          if (y != nullptr) {
            const float yy = DT<YT>::load(y + tp.at * W + c) + (y2 ? DT<YT>::load(y2 + tp.at * W + c) : 0.f);
            v += yy * inv[k] * nwc;
          }
        } else if (tp.kind == 2) {
          v = st[tp.at * W + c];
        }
        if (k == 0) v0 = v;
        if (cw != nullptr) acc += cw[(size_t)c * taps + (taps - 1 - k)] * v;
      }
    }
    if (y != nullptr) xs[(size_t)t * W + c] = v0;
    if (cw != nullptr) {
      DT<OT>::store(h + (size_t)t * W + c, v0 + acc);
      if (shift_state && taps > 1) {
        // one row per sequence (a decode step): this workgroup is the only reader of the sequence's
        // state, and a lane has read its column's old rows above, so it shifts the column here
        for (int i = 0; i + 2 < taps; ++i)
          st[(size_t)i * W + c] = (pos - (taps - 2 - i) >= 0) ? st[(size_t)(i + 1) * W + c] : 0.f;
        st[(size_t)(taps - 2) * W + c] = v0;
      }
    }
  }
}

// one workgroup per sequence: the last `keep` rows of its span (columns col_off .. col_off + C of
// x) become its state; a shorter span keeps the newest old rows
template <typename XT>
__global__ void __launch_bounds__(kThreads) conv_state_kernel(const XT* __restrict__ x, int stride, int col_off, int C,
                                                              float* __restrict__ state, int sub, int nsub, int keep,
                                                              const int* __restrict__ cu_q,
                                                              const int* __restrict__ start_pos,
                                                              const int* __restrict__ slots) {
  const int s = blockIdx.x;
  const int r0 = cu_q[s], n = cu_q[s + 1] - r0;
  if (n <= 0) return;
  float* st = state + ((size_t)slots[s] * nsub + sub) * keep * C;
  const int p0 = start_pos[s];
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float nv[kMaxTaps];
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
      nv[i] = 0.f;
      if (i < keep) {
        const int idx = n - keep + i;   // row of this span, or (< 0) a row of the old state
        if (idx >= 0) nv[i] = DT<XT>::load(x + (size_t)(r0 + idx) * stride + col_off + c);
        else if (p0 + idx >= 0) nv[i] = st[(size_t)(keep + idx) * C + c];
      }
    }
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i)
      if (i < keep) st[(size_t)i * C + c] = nv[i];
  }
}

// dynamic LDS: the biased query row [H * Dk], then the biased key row [G * Dk]
template <typename T>
__global__ void __launch_bounds__(kThreads) qkv_prep_wide_kernel(
    T* __restrict__ qo, const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off, int v_from_k,
    const float* __restrict__ qb, const float* __restrict__ kb, const float* __restrict__ qw,
    const float* __restrict__ kw, const float* __restrict__ freq, int R, float mag, const float* __restrict__ vfreq,
    float eps, const int64_t* __restrict__ positions, T* __restrict__ kc, T* __restrict__ vc,
    const int64_t* __restrict__ slot_mapping, int H, int G, int Dk, int Dv, int BS) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* pr = proj + (size_t)t * stride;
  const int nq = H * Dk, nk = G * Dk;
  float* qr = row;
  float* kr = row + nq;
  const float pos = (float)positions[t];
  const int64_t slot = slot_mapping[t];
  const size_t blk = (size_t)(slot / BS);
  const int boff = (int)(slot % BS);
  float ssq = 0.f, ssk = 0.f;
  for (int c = threadIdx.x; c < nq; c += blockDim.x) {
    const float v = DT<T>::load(pr + q_off + c) + (qb ? qb[c] : 0.f);
    qr[c] = v;
    ssq += v * v;
  }
  for (int c = threadIdx.x; c < nk; c += blockDim.x) {
    const float v = DT<T>::load(pr + k_off + c) + (kb ? kb[c] : 0.f);
    kr[c] = v;
    ssk += v * v;
    if (v_from_k) {     // the values are the keys as projected (Dv == Dk)
      const int g = c / Dk, d = c - g * Dk;
      DT<T>::store(vc + ((blk * G + g) * BS + boff) * Dv + d, v);
    }
  }
  const float iq = rsqrtf(rt::block_sum(ssq, scratch) / nq + eps);
  const float ik = rsqrtf(rt::block_sum(ssk, scratch) / nk + eps);
  __syncthreads();
  // every lane owns whole pairs: (i, i + R) for i < R, single entries from 2R on
  const int per = Dk - R;       // work items per head: R pairs + (Dk - 2R) singles
  for (int w = threadIdx.x; w < (H + G) * per; w += blockDim.x) {
    const int hh = w / per, i = w - hh * per;
    const bool isq = hh < H;
    const int head = isq ? hh : hh - H;
    const float* src = (isq ? qr : kr) + head * Dk;
    const float* wt = (isq ? qw : kw) + head * Dk;
    const float nrm = isq ? iq : ik;
    T* dst = isq ? qo + ((size_t)t * H + head) * Dk : kc + ((blk * G + head) * BS + boff) * Dk;
    if (i < R) {
      float sn, cs;
      sincosf(pos * freq[i], &sn, &cs);
      sn *= mag;
      cs *= mag;
      const float u = src[i] * nrm * wt[i], v = src[i + R] * nrm * wt[i + R];
      DT<T>::store(dst + i, u * cs - v * sn);
      DT<T>::store(dst + i + R, v * cs + u * sn);
    } else {
      const int d = i + R;
      DT<T>::store(dst + d, src[d] * nrm * wt[d]);
    }
  }
  if (!v_from_k) {
    const int RV = vfreq ? Dv / 2 : 0;
    const int perv = Dv - RV;
    for (int w = threadIdx.x; w < G * perv; w += blockDim.x) {
      const int g = w / perv, i = w - g * perv;
      const T* src = pr + v_off + g * Dv;
      T* dst = vc + ((blk * G + g) * BS + boff) * Dv;
      if (i < RV) {
        float sn, cs;
        sincosf(pos * vfreq[i], &sn, &cs);
        const float u = DT<T>::load(src + i), v = DT<T>::load(src + i + RV);
        DT<T>::store(dst + i, u * cs - v * sn);
        DT<T>::store(dst + i + RV, v * cs + u * sn);
      } else {
        const int d = i + RV;
        DT<T>::store(dst + d, DT<T>::load(src + d));
      }
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(kThreads) turn_back_kernel(T* __restrict__ out, int out_stride, int out_off,
                                                             const T* __restrict__ o, int H, int E,
                                                             const int64_t* __restrict__ positions,
                                                             const float* __restrict__ vfreq, float scale) {
  const int t = blockIdx.x;
  const float pos = -(float)positions[t];
  const int R = E / 2, per = E - R;
  for (int w = threadIdx.x; w < H * per; w += blockDim.x) {
    const int h = w / per, i = w - h * per;
    const T* src = o + ((size_t)t * H + h) * E;
    T* dst = out + (size_t)t * out_stride + out_off + h * E;
    if (i < R) {
      float sn, cs;
      sincosf(pos * vfreq[i], &sn, &cs);
      const float u = DT<T>::load(src + i), v = DT<T>::load(src + i + R);
      DT<T>::store(dst + i, (u * cs - v * sn) * scale);
      DT<T>::store(dst + i + R, (v * cs + u * sn) * scale);
    } else {
      DT<T>::store(dst + i + R, DT<T>::load(src + i + R) * scale);
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(kThreads) silu_cols_kernel(float* __restrict__ out, const T* __restrict__ proj,
                                                             int stride, int off, int n, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t r = i / n;
  out[i] = silu(DT<T>::load(proj + r * stride + off + (i - r * n)));
}

template <typename T>
__global__ void __launch_bounds__(kThreads) relu2_kernel(T* __restrict__ out, const T* __restrict__ a, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float v = fmaxf(DT<T>::load(a + i), 0.f);
  DT<T>::store(out + i, v * v);
}

// out [6][T][A * D] = r, k, v, w, a * u, u; one wave per head
template <typename T>
__global__ void __launch_bounds__(kThreads) removal_prep_kernel(
    float* __restrict__ out, const T* __restrict__ proj, int stride, int r_off, int k_off, int v_off, int a_off,
    const T* __restrict__ lw, const float* __restrict__ w0, const float* __restrict__ ab, int Tn, int A, int D) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const T* pr = proj + (size_t)t * stride;
  const size_t n = (size_t)A * D, plane = (size_t)Tn * n;
  const float kdec = -0.60653065971263342f;     // -e^(-1/2)
  for (int a = wave; a < A; a += nw) {
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float kv = DT<T>::load(pr + k_off + a * D + d);
      ss += kv * kv;
    }
    const float iu = rsqrtf(rt::wave_sum(ss) + 1e-6f);
    for (int d = lane; d < D; d += 64) {
      const int c = a * D + d;
      float* o = out + (size_t)t * n + c;
      const float kv = DT<T>::load(pr + k_off + c);
      const float u = kv * iu;
      o[0] = DT<T>::load(pr + r_off + c);
      o[plane] = kv;
      o[2 * plane] = DT<T>::load(pr + v_off + c);
      o[3 * plane] = __expf(kdec * sigm(DT<T>::load(lw + (size_t)t * n + c) + w0[c]));
      o[4 * plane] = sigm(DT<T>::load(pr + a_off + c) + ab[c]) * u;
      o[5 * plane] = u;
    }
  }
}

// dynamic LDS: z [C] (convolved, silu), then the unit factors of the G query heads and G key heads
template <typename T>
__global__ void __launch_bounds__(1024) delta_prep_kernel(
    float* __restrict__ five, float* __restrict__ vout, const T* __restrict__ proj, int stride, int q_off, int b_off,
    int a_off, const float* __restrict__ cw, float* __restrict__ state, const float* __restrict__ neg_rate,
    const float* __restrict__ dt_bias, int Tn, int A, int G, int D, int E, int taps, int keep,
    const int* __restrict__ row_seq, const int64_t* __restrict__ positions, const int* __restrict__ start_pos,
    const int* __restrict__ slots, int shift_state) {
  extern __shared__ float z[];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int C = 2 * G * D + A * E;
  float* unit = z + C;          // [2 * G]
  const int s = row_seq[t];
  const int64_t pos = positions[t];
  const int local = (int)(pos - start_pos[s]);
  float* st = state + (size_t)slots[s] * keep * C;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float acc = 0.f, v0 = 0.f;
    for (int k = 0; k < taps; ++k) {
      const Tap tp = tap_of(k, t, local, pos, taps);
      float v = 0.f;
      if (tp.kind == 1) v = DT<T>::load(proj + tp.at * stride + q_off + c);
      else if (tp.kind == 2) v = st[tp.at * C + c];
      if (k == 0) v0 = v;
      acc += cw[(size_t)c * taps + (taps - 1 - k)] * v;
    }
    z[c] = silu(acc);
    if (shift_state && taps > 1) {
      for (int i = 0; i + 2 < taps; ++i)
        st[(size_t)i * C + c] = (pos - (taps - 2 - i) >= 0) ? st[(size_t)(i + 1) * C + c] : 0.f;
      st[(size_t)(taps - 2) * C + c] = v0;
    }
  }
  __syncthreads();
  for (int j = wave; j < 2 * G; j += nw) {     // q heads, then k heads
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) ss += z[j * D + d] * z[j * D + d];
    const float iv = rsqrtf(rt::wave_sum(ss) + 1e-6f);
    if (lane == 0) unit[j] = iv;
  }
  __syncthreads();
  const size_t n = (size_t)A * D, plane = (size_t)Tn * n;
  const int rep = A / G;
  const float qs = rsqrtf((float)D);
  const T* pr = proj + (size_t)t * stride;
  for (int a = wave; a < A; a += nw) {
    const int g = a / rep;
    const float beta = sigm(DT<T>::load(pr + b_off + a));
    const float xa = DT<T>::load(pr + a_off + a) + dt_bias[a];
    const float sp = xa > 20.f ? xa : log1pf(__expf(xa));
    const float gd = __expf(neg_rate[a] * sp);
    for (int d = lane; d < D; d += 64) {
      float* o = five + (size_t)t * n + a * D + d;
      const float qv = z[g * D + d] * unit[g] * qs;
      const float kv = z[(G + g) * D + d] * unit[G + g];
      o[0] = qv;
      o[plane] = beta * kv;
      o[2 * plane] = gd;
      o[3 * plane] = gd * beta * kv;
      o[4 * plane] = kv;
    }
  }
  for (int c = threadIdx.x; c < A * E; c += blockDim.x) vout[(size_t)t * A * E + c] = z[2 * G * D + c];
}

// o [T, C] fp32: segments of `span` entries are divided by their RMS; wmod = entries of the weight
template <typename OT, typename GT>
__global__ void __launch_bounds__(kThreads) head_norm_gate_kernel(
    OT* __restrict__ out, int out_stride, int out_off, const float* __restrict__ o, const float* __restrict__ w, int wmod,
    int span, const GT* __restrict__ gate, int gate_stride, int gate_off, int act, float eps, float scale, int C) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const float* orow = o + (size_t)t * C;
  const GT* grow = gate + (size_t)t * gate_stride + gate_off;
  OT* dst = out + (size_t)t * out_stride + out_off;
  if (span == C) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < C; c += blockDim.x) ss += orow[c] * orow[c];
    const float iv = rsqrtf(rt::block_sum(ss, scratch) / C + eps);
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
      const float g = DT<GT>::load(grow + c);
      DT<OT>::store(dst + c, orow[c] * iv * w[c % wmod] * (act ? silu(g) : sigm(g)) * scale);
    }
    return;
  }
  for (int h = wave; h < C / span; h += nw) {
    float ss = 0.f;
    for (int d = lane; d < span; d += 64) ss += orow[h * span + d] * orow[h * span + d];
    const float iv = rsqrtf(rt::wave_sum(ss) / span + eps);
    for (int d = lane; d < span; d += 64) {
      const int c = h * span + d;
      const float g = DT<GT>::load(grow + c);
      DT<OT>::store(dst + c, orow[c] * iv * w[c % wmod] * (act ? silu(g) : sigm(g)) * scale);
    }
  }
}

}  // namespace

void launch_canon_add(void* h, float* xs, const float* x, const void* y, const void* y2, const float* nw, float eps,
                      const float* cw, float* state, int sub, int nsub, const int* row_seq, const int64_t* positions,
                      const int* start_pos, const int* slots, int T, int W, int taps, int keep, bool out_bf, bool y_bf,
                      bool shift_state, hipStream_t stream) {
  if (T <= 0) return;
  // about one entry per lane (64 .. 1024 lanes): a row's loads leave together, which is what a
  // decode step of a few rows waits for
  const int th = W >= 1024 ? 1024 : W <= 64 ? 64 : (W + 63) / 64 * 64;
#define RT_CA2(OT, YT, TP)                                                                                             \
  canon_add_kernel<OT, YT, TP><<<T, th, 0, stream>>>((OT*)h, xs, x, (const YT*)y, (const YT*)y2, nw, eps, cw,     \
                                                           state, sub, nsub, row_seq, positions, start_pos, slots, W,    \
                                                           taps, keep, shift_state ? 1 : 0)
#define RT_CA(OT, YT)                                                                                                  \
  do {                                                                                                                 \
    const int tp = cw == nullptr ? 0 : taps;                                                                           \
    if (tp == 0) RT_CA2(OT, YT, 0); else if (tp == 1) RT_CA2(OT, YT, 1); else if (tp == 2) RT_CA2(OT, YT, 2);          \
    else if (tp == 3) RT_CA2(OT, YT, 3); else if (tp == 4) RT_CA2(OT, YT, 4); else RT_CA2(OT, YT, kMaxTaps);           \
  } while (0)
  if (out_bf) {
    if (y_bf) RT_CA(uint16_t, uint16_t); else RT_CA(uint16_t, float);
  } else {
    if (y_bf) RT_CA(float, uint16_t); else RT_CA(float, float);
  }
#undef RT_CA
#undef RT_CA2
}

void launch_conv_state(const void* x, int stride, int col_off, int C, float* state, int sub, int nsub, int keep,
                       const int* cu_q, const int* start_pos, const int* slots, int S, bool bf, hipStream_t stream) {
  if (S <= 0) return;
  if (bf) conv_state_kernel<uint16_t><<<S, kThreads, 0, stream>>>((const uint16_t*)x, stride, col_off, C, state, sub, nsub,
                                                                   keep, cu_q, start_pos, slots);
  else conv_state_kernel<float><<<S, kThreads, 0, stream>>>((const float*)x, stride, col_off, C, state, sub, nsub, keep,
                                                            cu_q, start_pos, slots);
}

int launch_qkv_prep_wide(void* q, const void* proj, int stride, int q_off, int k_off, int v_off, bool v_from_k,
                         const float* qb, const float* kb, const float* qw, const float* kw, const float* freq, int R,
                         float mag, const float* vfreq, float eps, const int64_t* positions, void* kc, void* vc,
                         const int64_t* slot_mapping, int T, int H, int G, int Dk, int Dv, int BS, bool bf,
                         hipStream_t stream) {
  if (T <= 0) return 0;
  const size_t shm = sizeof(float) * (size_t)(H + G) * Dk;
  if (shm > 150 * 1024) return -1;
#define RT_QW(TT)                                                                                                      \
  do {                                                                                                                 \
    auto kern = qkv_prep_wide_kernel<TT>;                                                                              \
    if (shm > 48 * 1024 &&                                                                                             \
        hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm) != hipSuccess)    \
      return -2;                                                                                                       \
    kern<<<T, kThreads, shm, stream>>>((TT*)q, (const TT*)proj, stride, q_off, k_off, v_off, v_from_k ? 1 : 0, qb, kb,  \
                                       qw, kw, freq, R, mag, vfreq, eps, positions, (TT*)kc, (TT*)vc, slot_mapping, H,  \
                                       G, Dk, Dv, BS);                                                                 \
  } while (0)
  if (bf) RT_QW(uint16_t); else RT_QW(float);
#undef RT_QW
  return 0;
}

void launch_turn_back(void* out, int out_stride, int out_off, const void* o, int T, int H, int E,
                      const int64_t* positions, const float* vfreq, float scale, bool bf, hipStream_t stream) {
  if (T <= 0) return;
  if (bf) turn_back_kernel<uint16_t><<<T, kThreads, 0, stream>>>((uint16_t*)out, out_stride, out_off, (const uint16_t*)o, H,
                                                                  E, positions, vfreq, scale);
  else turn_back_kernel<float><<<T, kThreads, 0, stream>>>((float*)out, out_stride, out_off, (const float*)o, H, E,
                                                           positions, vfreq, scale);
}

void launch_silu_cols(float* out, const void* proj, int stride, int off, int n, int T, bool bf, hipStream_t stream) {
  const int64_t total = (int64_t)T * n;
  if (total <= 0) return;
  const int blocks = (int)((total + kThreads - 1) / kThreads);
  if (bf) silu_cols_kernel<uint16_t><<<blocks, kThreads, 0, stream>>>(out, (const uint16_t*)proj, stride, off, n, total);
  else silu_cols_kernel<float><<<blocks, kThreads, 0, stream>>>(out, (const float*)proj, stride, off, n, total);
}

void launch_relu2(void* out, const void* a, int64_t total, bool bf, hipStream_t stream) {
  if (total <= 0) return;
  const int blocks = (int)((total + kThreads - 1) / kThreads);
  if (bf) relu2_kernel<uint16_t><<<blocks, kThreads, 0, stream>>>((uint16_t*)out, (const uint16_t*)a, total);
  else relu2_kernel<float><<<blocks, kThreads, 0, stream>>>((float*)out, (const float*)a, total);
}

void launch_removal_prep(float* out, const void* proj, int stride, int r_off, int k_off, int v_off, int a_off,
                         const void* lw, const float* w0, const float* ab, int T, int A, int D, bool bf,
                         hipStream_t stream) {
  if (T <= 0) return;
  if (bf) removal_prep_kernel<uint16_t><<<T, kThreads, 0, stream>>>(out, (const uint16_t*)proj, stride, r_off, k_off, v_off,
                                                                     a_off, (const uint16_t*)lw, w0, ab, T, A, D);
  else removal_prep_kernel<float><<<T, kThreads, 0, stream>>>(out, (const float*)proj, stride, r_off, k_off, v_off, a_off,
                                                              (const float*)lw, w0, ab, T, A, D);
}

int launch_delta_prep(float* five, float* vout, const void* proj, int stride, int q_off, int b_off, int a_off,
                      const float* cw, float* state, const float* neg_rate, const float* dt_bias, int T, int A, int G,
                      int D, int E, int taps, int keep, const int* row_seq, const int64_t* positions,
                      const int* start_pos, const int* slots, bool shift_state, bool bf, hipStream_t stream) {
  if (T <= 0) return 0;
  const size_t shm = sizeof(float) * ((size_t)2 * G * D + (size_t)A * E + 2 * G);
  if (shm > 150 * 1024 || taps > kMaxTaps) return -1;
  const int C = 2 * G * D + A * E;
  const int th = C >= 1024 ? 1024 : C <= 256 ? 256 : (C + 63) / 64 * 64;
#define RT_DP(TT)                                                                                                      \
  do {                                                                                                                 \
    auto kern = delta_prep_kernel<TT>;                                                                                 \
    if (shm > 48 * 1024 &&                                                                                             \
        hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm) != hipSuccess)    \
      return -2;                                                                                                       \
    kern<<<T, th, shm, stream>>>(five, vout, (const TT*)proj, stride, q_off, b_off, a_off, cw, state, neg_rate,         \
                                       dt_bias, T, A, G, D, E, taps, keep, row_seq, positions, start_pos, slots,       \
                                       shift_state ? 1 : 0);                                                           \
  } while (0)
  if (bf) RT_DP(uint16_t); else RT_DP(float);
#undef RT_DP
  return 0;
}

void launch_head_norm_gate(void* out, int out_stride, int out_off, const float* o, const float* w, int wmod, int span,
                           const void* gate, int gate_stride, int gate_off, int act, float eps, float scale, int T, int C,
                           bool out_bf, bool gate_bf, hipStream_t stream) {
  if (T <= 0) return;
#define RT_HN(OT, GT)                                                                                                  \
  head_norm_gate_kernel<OT, GT><<<T, kThreads, 0, stream>>>((OT*)out, out_stride, out_off, o, w, wmod, span,           \
                                                            (const GT*)gate, gate_stride, gate_off, act, eps, scale, C)
  if (out_bf) {
    if (gate_bf) RT_HN(uint16_t, uint16_t); else RT_HN(uint16_t, float);
  } else {
    if (gate_bf) RT_HN(float, uint16_t); else RT_HN(float, float);
  }
#undef RT_HN
}
