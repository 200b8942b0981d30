// H8: the wkv recurrence (linear attention with a per-token, per-channel decay), fused with what
// follows it per head. All math fp32; tensors bf16 (uint16_t storage) or fp32 as templated.
//
//   per head, state S [D keys][D values] fp32, from the sequence's slot (zero at position 0):
//     decay_t[i] = exp(-exp(lw_t[i] + w0[i]))
//     o_t[j]     = sum_i r_t[i] * (S[i][j] + u[i] k_t[i] v_t[j])
//     S[i][j]    = decay_t[i] * S[i][j] + k_t[i] v_t[j]
//     out_t[j]   = o_t[j] / rms_j(o_t) * norm_w[j] * silu(g_t[j])
//
// One workgroup per (sequence, head); thread j owns value column j and keeps S[.][j] in registers
// (DB = the power of two >= D, at least 64; rows i >= D are never touched). r, k and the decay of a
// token are staged in LDS (two buffers, one barrier a token) and read by every thread.
//
// Long spans run in three launches over chunks of kWkvChunk rows, like the minGRU scan: (A) every
// chunk alone from S = 0: its end state E and its decay product Pd[i]; (B) per (sequence, head),
// chunk by chunk: the state each chunk starts from (carry = Pd * carry + E) and the sequence's new
// state; (C) every chunk again from its true start state, writing the outputs. No division by a
// decay product anywhere, so small decays are harmless.
#include "../common.h"

namespace {

using rt::DT;

constexpr int kWkvChunk = 64;

RT_DEVICE float sigm(float v) { return 1.0f / (1.0f + expf(-v)); }

// MODE 0: whole spans, state in and out of the slots. MODE 1: phase A. MODE 3: phase C.
template <typename T, int DB, int MODE>
__global__ void __launch_bounds__(DB) wkv_scan_kernel(
    T* __restrict__ out, const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ g, const T* __restrict__ lw, int stride, int lw_stride, const float* __restrict__ w0,
    const float* __restrict__ u, const float* __restrict__ norm_w, float* __restrict__ state,
    const int* __restrict__ cu_q, const int* __restrict__ start_pos, const int* __restrict__ slots,
    const int* __restrict__ chunks, float* __restrict__ ws_e, float* __restrict__ ws_p,
    const float* __restrict__ ws_in, int H, int D, float eps) {
  __shared__ float sr[2][DB], sk[2][DB], sw[2][DB], su[DB], red[2][DB / 64];
  const int j = threadIdx.x, lane = j & 63, wid = j >> 6;
  const int h = blockIdx.y;
  int s, r0, r1;
  if (MODE == 0) {
    s = blockIdx.x;
    r0 = cu_q[s];
    r1 = cu_q[s + 1];
  } else {
    s = chunks[2 * blockIdx.x];
    r0 = chunks[2 * blockIdx.x + 1];
    r1 = min(r0 + kWkvChunk, cu_q[s + 1]);
  }
  if (r1 <= r0) return;
  const bool on = j < D;
  const size_t DD = (size_t)D * D;
  float S[DB];
  float* st = nullptr;
  if (MODE == 0) {
    st = state + ((size_t)slots[s] * H + h) * DD;
    const bool keep = start_pos[s] > 0;
#pragma unroll
    for (int i = 0; i < DB; ++i) S[i] = (keep && on && i < D) ? st[(size_t)i * D + j] : 0.f;
  } else if (MODE == 3) {
    const float* in = ws_in + ((size_t)blockIdx.x * H + h) * DD;
#pragma unroll
    for (int i = 0; i < DB; ++i) S[i] = (on && i < D) ? in[(size_t)i * D + j] : 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < DB; ++i) S[i] = 0.f;
  }
  const int col = h * D + j;
  su[j] = on ? u[col] : 0.f;
  const float w0j = on ? w0[col] : 0.f, nwj = on && MODE != 1 ? norm_w[col] : 0.f;
  float pd = 1.f;
  for (int t = r0; t < r1; ++t) {
    const int b = (t - r0) & 1;
    float vj = 0.f, gj = 0.f;
    if (on) {
      const size_t at = (size_t)t * stride + col;
      const float dec = expf(-expf(DT<T>::load(lw + (size_t)t * lw_stride + col) + w0j));
      sr[b][j] = MODE == 1 ? 0.f : DT<T>::load(r + at);
      sk[b][j] = DT<T>::load(k + at);
      sw[b][j] = dec;
      vj = DT<T>::load(v + at);
      if (MODE != 1) gj = DT<T>::load(g + at);
      pd *= dec;
    }
    __syncthreads();        // the token's r, k, decay are staged (the other buffer's readers are done)
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < DB; ++i) {
      if (i < D) {
        const float kv = sk[b][i] * vj;
        if (MODE != 1) acc += sr[b][i] * (S[i] + su[i] * kv);
        S[i] = sw[b][i] * S[i] + kv;
      }
    }
    if (MODE != 1) {
      float ss = rt::wave_sum(on ? acc * acc : 0.f);
      if (DB > 64) {
        if (lane == 0) red[b][wid] = ss;
        __syncthreads();
        ss = 0.f;
#pragma unroll
        for (int q = 0; q < DB / 64; ++q) ss += red[b][q];
      }
      if (on) DT<T>::store(out + (size_t)t * stride + col, acc / sqrtf(ss / (float)D + eps) * nwj * (gj * sigm(gj)));
    }
  }
  if (!on) return;
  if (MODE == 0) {
#pragma unroll
    for (int i = 0; i < DB; ++i)
      if (i < D) st[(size_t)i * D + j] = S[i];
  } else if (MODE == 1) {
    float* e = ws_e + ((size_t)blockIdx.x * H + h) * DD;
#pragma unroll
    for (int i = 0; i < DB; ++i)
      if (i < D) e[(size_t)i * D + j] = S[i];
    ws_p[((size_t)blockIdx.x * H + h) * D + j] = pd;
  }
}

// phase B: grid (sequences, heads, row blocks of the state), thread = one (i, j) entry of S
__global__ void __launch_bounds__(256) wkv_carry_kernel(const float* __restrict__ ws_e, const float* __restrict__ ws_p,
                                                        float* __restrict__ ws_in, float* __restrict__ state,
                                                        const int* __restrict__ seq_chunk0,
                                                        const int* __restrict__ start_pos, const int* __restrict__ slots,
                                                        int H, int D) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * blockDim.x + threadIdx.x;      // entry i * D + j
  const int DD = D * D;
  const int k0 = seq_chunk0[s], k1 = seq_chunk0[s + 1];
  if (e >= DD || k1 <= k0) return;
  const int i = e / D;
  float* st = state + ((size_t)slots[s] * H + h) * DD + e;
  float S = start_pos[s] > 0 ? *st : 0.f;
  for (int c = k0; c < k1; ++c) {
    const size_t at = (size_t)c * H + h;
    ws_in[at * DD + e] = S;
    S = ws_p[at * D + i] * S + ws_e[at * DD + e];
  }
  *st = S;
}

}  // namespace

int wkv_scan_chunk() { return kWkvChunk; }

// chunks == nullptr: one launch over whole spans (grid S x H). Otherwise the three launches over
// `n_chunks` chunks; ws holds n_chunks * H * (2 * D * D + D) floats.
int launch_wkv_scan(void* out, const void* r, const void* k, const void* v, const void* g, const void* lw, int stride,
                    int lw_stride, const float* w0, const float* u, const float* norm_w, float* state, const int* cu_q,
                    const int* start_pos, const int* slots, int S, int H, int D, float eps, const int* chunks,
                    int n_chunks, const int* seq_chunk0, float* ws, bool bf, hipStream_t stream) {
  if (S <= 0 || H <= 0) return 0;
  if (D < 1 || D > 256) return -1;
  const int db = D <= 64 ? 64 : D <= 128 ? 128 : 256;
  const size_t DD = (size_t)D * D;
  float* ws_e = ws;
  float* ws_in = ws ? ws + (size_t)n_chunks * H * DD : nullptr;
  float* ws_p = ws ? ws + 2 * (size_t)n_chunks * H * DD : nullptr;
#define RT_WKV(TT, DBV, MODE, GRID)                                                                                  \
  wkv_scan_kernel<TT, DBV, MODE><<<GRID, DBV, 0, stream>>>((TT*)out, (const TT*)r, (const TT*)k, (const TT*)v,       \
                                                           (const TT*)g, (const TT*)lw, stride, lw_stride, w0, u,    \
                                                           norm_w, state, cu_q, start_pos, slots, chunks, ws_e,      \
                                                           ws_p, ws_in, H, D, eps)
#define RT_WKV_T(DBV, MODE, GRID)                                                                                    \
  do {                                                                                                               \
    if (bf) RT_WKV(uint16_t, DBV, MODE, GRID); else RT_WKV(float, DBV, MODE, GRID);                                  \
  } while (0)
#define RT_WKV_D(MODE, GRID)                                                                                         \
  do {                                                                                                               \
    if (db == 64) RT_WKV_T(64, MODE, GRID); else if (db == 128) RT_WKV_T(128, MODE, GRID);                           \
    else RT_WKV_T(256, MODE, GRID);                                                                                  \
  } while (0)
  if (chunks == nullptr) {
    RT_WKV_D(0, dim3(S, H));
    return 0;
  }
  if (n_chunks <= 0) return 0;
  RT_WKV_D(1, dim3(n_chunks, H));
  wkv_carry_kernel<<<dim3(S, H, (unsigned)((DD + 255) / 256)), 256, 0, stream>>>(ws_e, ws_p, ws_in, state, seq_chunk0,
                                                                                 start_pos, slots, H, D);
  RT_WKV_D(3, dim3(n_chunks, H));
#undef RT_WKV
#undef RT_WKV_T
#undef RT_WKV_D
  return 0;
}
