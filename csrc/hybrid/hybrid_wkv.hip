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
// (DB = the power of two >= D, at least 64; rows i >= D are never touched). The rows of a span are
// taken in blocks of up to SB tokens: every thread first copies its column of r, k, v, the gate and
// the decay of the whole block to LDS (independent loads, all in flight together), then the
// recurrence runs over the block reading LDS only — no global load and, for heads of up to 64
// columns (one wave), no barrier inside the token loop.
//
// Long spans run in three launches over chunks of kWkvChunk rows, like the minGRU scan: (A) every
// chunk alone from S = 0: its end state E and its decay product Pd[i]; (B) per (sequence, head),
// chunk by chunk: the state each chunk starts from (carry = Pd * carry + E, written over E) and the
// sequence's new state; (C) every chunk again from its true start state, writing the outputs. No
// division by a decay product anywhere, so small decays are harmless.
#include "../common.h"

namespace {

using rt::DT;

constexpr int kWkvChunk = 32;

RT_DEVICE float sigm(float v) { return 1.0f / (1.0f + expf(-v)); }

// tokens staged at a time: 5 arrays of SB x DB floats (40 KB at DB = 64, 80 KB at 128 and 256)
template <int DB> constexpr int stage_rows() { return DB <= 64 ? 32 : DB <= 128 ? 32 : 16; }
template <int DB> constexpr size_t wkv_lds_bytes() { return sizeof(float) * ((size_t)5 * stage_rows<DB>() * DB + DB + 8); }

// MODE 0: whole spans, state in and out of the slots. MODE 1: phase A. MODE 3: phase C.
template <typename T, int DB, int MODE>
__global__ void __launch_bounds__(DB) wkv_scan_kernel(
    T* __restrict__ out, const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ g, const T* __restrict__ lw, int stride, int lw_stride, const float* __restrict__ w0,
    const float* __restrict__ u, const float* __restrict__ norm_w, float* __restrict__ state,
    const int* __restrict__ cu_q, const int* __restrict__ start_pos, const int* __restrict__ slots,
    const int* __restrict__ chunks, float* __restrict__ ws_e, float* __restrict__ ws_p, int H, int D, float eps) {
  constexpr int SB = stage_rows<DB>();
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* sr = lds;                  // [SB][DB] each
  float* sk = sr + SB * DB;
  float* sw = sk + SB * DB;
  float* sv = sw + SB * DB;
  float* sg = sv + SB * DB;
  float* su = sg + SB * DB;         // [DB]
  float* red = su + DB;             // [2][4]
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
    const float* in = ws_e + ((size_t)blockIdx.x * H + h) * DD;      // phase B left the start state here
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
  for (int t0 = r0; t0 < r1; t0 += SB) {
    const int n = min(SB, r1 - t0);
    __syncthreads();        // the previous block's readers are done
    if (on) {
#pragma unroll 8
      for (int tt = 0; tt < n; ++tt) {
        const size_t at = (size_t)(t0 + tt) * stride + col;
        const float dec = expf(-expf(DT<T>::load(lw + (size_t)(t0 + tt) * lw_stride + col) + w0j));
        sk[tt * DB + j] = DT<T>::load(k + at);
        sv[tt * DB + j] = DT<T>::load(v + at);
        sw[tt * DB + j] = dec;
        if (MODE != 1) {
          sr[tt * DB + j] = DT<T>::load(r + at);
          sg[tt * DB + j] = DT<T>::load(g + at);
        }
        pd *= dec;
      }
    } else {
      // key channels past D: zeros, so the token loop runs over all DB rows without a test and
      // those rows of S stay zero
      for (int tt = 0; tt < n; ++tt) {
        sk[tt * DB + j] = 0.f;
        sw[tt * DB + j] = 0.f;
        sv[tt * DB + j] = 0.f;
        if (MODE != 1) {
          sr[tt * DB + j] = 0.f;
          sg[tt * DB + j] = 0.f;
        }
      }
    }
    __syncthreads();        // the block's r, k, decay are staged
    for (int tt = 0; tt < n; ++tt) {
      // rows of the block as 16-byte LDS reads (every lane reads the same address: a broadcast)
      const float4* kr = reinterpret_cast<const float4*>(sk + tt * DB);
      const float4* rr = reinterpret_cast<const float4*>(sr + tt * DB);
      const float4* wr = reinterpret_cast<const float4*>(sw + tt * DB);
      const float4* ur = reinterpret_cast<const float4*>(su);
      const float vj = sv[tt * DB + j];
      float a4[4] = {0.f, 0.f, 0.f, 0.f};     // four partial sums: no 64-long dependent chain
#pragma unroll
      for (int q = 0; q < DB / 4; ++q) {
        const float4 k4 = kr[q], w4 = wr[q];
        const float kv0 = k4.x * vj, kv1 = k4.y * vj, kv2 = k4.z * vj, kv3 = k4.w * vj;
        if (MODE != 1) {
          const float4 r4 = rr[q], u4 = ur[q];
          a4[0] += r4.x * (S[4 * q] + u4.x * kv0);
          a4[1] += r4.y * (S[4 * q + 1] + u4.y * kv1);
          a4[2] += r4.z * (S[4 * q + 2] + u4.z * kv2);
          a4[3] += r4.w * (S[4 * q + 3] + u4.w * kv3);
        }
        S[4 * q] = w4.x * S[4 * q] + kv0;
        S[4 * q + 1] = w4.y * S[4 * q + 1] + kv1;
        S[4 * q + 2] = w4.z * S[4 * q + 2] + kv2;
        S[4 * q + 3] = w4.w * S[4 * q + 3] + kv3;
      }
      const float acc = (a4[0] + a4[1]) + (a4[2] + a4[3]);
      if (MODE != 1) {
        float ss = rt::wave_sum(on ? acc * acc : 0.f);
        if (DB > 64) {
          const int b = tt & 1;
          if (lane == 0) red[b * 4 + wid] = ss;
          __syncthreads();
          ss = 0.f;
#pragma unroll
          for (int q = 0; q < DB / 64; ++q) ss += red[b * 4 + q];
        }
        const float gj = sg[tt * DB + j];
        if (on)
          DT<T>::store(out + (size_t)(t0 + tt) * stride + col, acc / sqrtf(ss / (float)D + eps) * nwj * (gj * sigm(gj)));
      }
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

// phase B: grid (sequences, heads, row blocks of the state), thread = one (i, j) entry of S; every
// chunk's end state in ws_e is replaced by the state the chunk starts from
__global__ void __launch_bounds__(256) wkv_carry_kernel(float* __restrict__ ws_e, const float* __restrict__ ws_p,
                                                        float* __restrict__ state, const int* __restrict__ seq_chunk0,
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
    const float E = ws_e[at * DD + e];
    ws_e[at * DD + e] = S;
    S = ws_p[at * D + i] * S + E;
  }
  *st = S;
}

template <typename T, int DB, int MODE>
int launch_one(dim3 grid, hipStream_t stream, T* out, const T* r, const T* k, const T* v, const T* g, const T* lw,
               int stride, int lw_stride, const float* w0, const float* u, const float* norm_w, float* state,
               const int* cu_q, const int* start_pos, const int* slots, const int* chunks, float* ws_e, float* ws_p, int H,
               int D, float eps) {
  auto kern = wkv_scan_kernel<T, DB, MODE>;
  const size_t shm = wkv_lds_bytes<DB>();
  if (shm > 48 * 1024 &&
      hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm) != hipSuccess)
    return -2;
  kern<<<grid, DB, shm, stream>>>(out, r, k, v, g, lw, stride, lw_stride, w0, u, norm_w, state, cu_q, start_pos, slots,
                                  chunks, ws_e, ws_p, H, D, eps);
  return 0;
}

template <typename T, int MODE>
int launch_mode(int db, dim3 grid, hipStream_t stream, void* out, const void* r, const void* k, const void* v,
                const void* g, const void* lw, int stride, int lw_stride, const float* w0, const float* u,
                const float* norm_w, float* state, const int* cu_q, const int* start_pos, const int* slots,
                const int* chunks, float* ws_e, float* ws_p, int H, int D, float eps) {
#define RT_WKV(DBV)                                                                                                   \
  launch_one<T, DBV, MODE>(grid, stream, (T*)out, (const T*)r, (const T*)k, (const T*)v, (const T*)g, (const T*)lw,   \
                           stride, lw_stride, w0, u, norm_w, state, cu_q, start_pos, slots, chunks, ws_e, ws_p, H, D, eps)
  if (db == 64) return RT_WKV(64);
  if (db == 128) return RT_WKV(128);
  return RT_WKV(256);
#undef RT_WKV
}

}  // namespace

int wkv_scan_chunk() { return kWkvChunk; }

// chunks == nullptr: one launch over whole spans (grid S x H). Otherwise the three launches over
// `n_chunks` chunks; ws holds n_chunks * H * (D * D + D) floats.
int launch_wkv_scan(void* out, const void* r, const void* k, const void* v, const void* g, const void* lw, int stride,
                    int lw_stride, const float* w0, const float* u, const float* norm_w, float* state, const int* cu_q,
                    const int* start_pos, const int* slots, int S, int H, int D, float eps, const int* chunks,
                    int n_chunks, const int* seq_chunk0, float* ws, bool bf, hipStream_t stream) {
  if (S <= 0 || H <= 0) return 0;
  if (D < 1 || D > 256) return -1;
  const int db = D <= 64 ? 64 : D <= 128 ? 128 : 256;
  const size_t DD = (size_t)D * D;
  float* ws_e = ws;
  float* ws_p = ws ? ws + (size_t)n_chunks * H * DD : nullptr;
#define RT_WKV_M(MODE, GRID)                                                                                          \
  (bf ? launch_mode<uint16_t, MODE>(db, GRID, stream, out, r, k, v, g, lw, stride, lw_stride, w0, u, norm_w, state,   \
                                    cu_q, start_pos, slots, chunks, ws_e, ws_p, H, D, eps)                            \
      : launch_mode<float, MODE>(db, GRID, stream, out, r, k, v, g, lw, stride, lw_stride, w0, u, norm_w, state, cu_q, \
                                 start_pos, slots, chunks, ws_e, ws_p, H, D, eps))
  if (chunks == nullptr) return RT_WKV_M(0, dim3(S, H));
  if (n_chunks <= 0) return 0;
  int rc = RT_WKV_M(1, dim3(n_chunks, H));
  if (rc) return rc;
  wkv_carry_kernel<<<dim3(S, H, (unsigned)((DD + 255) / 256)), 256, 0, stream>>>(ws_e, ws_p, state, seq_chunk0, start_pos,
                                                                                 slots, H, D);
  return RT_WKV_M(3, dim3(n_chunks, H));
#undef RT_WKV_M
}
