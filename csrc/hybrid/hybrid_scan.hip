// C5: matrix-state recurrence, fp32 throughout. Per sequence and head a D x E state S:
//
//   s = b_t^T S ;  S <- diag(w_t) S - a_t s^T + k_t v_t^T ;  o_t = S^T q_t
//
// (w: a stream per key channel, or one constant per head; a / b: optional removal streams.) This
// covers a constant-decay linear attention (no a / b), a generalized delta rule (a = rate * unit
// key, b = unit key) and a gated delta rule (w = g, a = g beta k, b = k, k <- beta k).
//
// The columns of S are independent, so a lane owns DR rows of ONE column in registers and the token
// loop needs no LDS traffic for the state: P = D / DR adjacent lanes share a column and add their
// partial dot products with P - 1 xor shuffles. One workgroup of 256 lanes = (sequence, head,
// 256 / P columns); tokens are staged through LDS in chunks of TT (all streams of the head, padded
// to P * DR rows with zeros, plus the chunk's value columns), the chunk's outputs leave through
// LDS so that the global writes are whole lines. The state is kept column by column,
// [slot][head][E][D], so that a lane's rows are contiguous.
#include "../common.h"

namespace {

constexpr int kScanThreads = 256;

template <int DR, bool HAS_W, bool HAS_AB>
__global__ void __launch_bounds__(kScanThreads) state_scan_kernel(
    float* __restrict__ out, const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ w, const float* __restrict__ a, const float* __restrict__ b, int sq, int sk, int sv, int sw,
    int sa, int sb, const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ start_pos, const int* __restrict__ slots, int A, int D, int E, int P, int TT) {
  extern __shared__ float lds[];
  constexpr int NS = 2 + (HAS_W ? 1 : 0) + (HAS_AB ? 2 : 0);
  const int seq = blockIdx.x, head = blockIdx.y;
  const int CB = kScanThreads / P, Dp = P * DR;
  const int cl = threadIdx.x / P, part = threadIdx.x - cl * P;
  const int col = blockIdx.z * CB + cl;
  const int r0 = cu_q[seq], n = cu_q[seq + 1] - r0;
  if (n <= 0) return;
  float* str = lds;                       // [TT][NS][Dp]: q, k, (w), (a, b)
  float* vs = str + (size_t)TT * NS * Dp; // [TT][CB]
  float* os = vs + (size_t)TT * CB;       // [TT][CB]
  const int row_lo = part * DR;
  const bool live = col < E;
  float S[DR];
  float* sp = state + (((size_t)slots[seq] * A + head) * E + (live ? col : 0)) * D + row_lo;
  const bool cont = start_pos[seq] > 0;
#pragma unroll
  for (int i = 0; i < DR; ++i) S[i] = (cont && live && row_lo + i < D) ? sp[i] : 0.f;
  const float dconst = HAS_W ? 1.f : decay[head];
  const float* src[NS];
  int strides[NS];
  {
    int j = 0;
    src[j] = q; strides[j++] = sq;
    src[j] = k; strides[j++] = sk;
    if (HAS_W) { src[j] = w; strides[j++] = sw; }
    if (HAS_AB) { src[j] = a; strides[j++] = sa; src[j] = b; strides[j++] = sb; }
  }
  for (int c0 = 0; c0 < n; c0 += TT) {
    const int nt = min(TT, n - c0);
    __syncthreads();      // the previous chunk's readers are done
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      const float* base = src[j] + (size_t)(r0 + c0) * strides[j] + head * D;
      for (int i = threadIdx.x; i < nt * Dp; i += kScanThreads) {
        const int tok = i / Dp, r = i - tok * Dp;
        str[((size_t)tok * NS + j) * Dp + r] = r < D ? base[(size_t)tok * strides[j] + r] : 0.f;
      }
    }
    for (int i = threadIdx.x; i < nt * CB; i += kScanThreads) {
      const int tok = i / CB, c = i - tok * CB;
      const int gc = blockIdx.z * CB + c;
      vs[i] = gc < E ? v[(size_t)(r0 + c0 + tok) * sv + head * E + gc] : 0.f;
    }
    __syncthreads();
    for (int tok = 0; tok < nt; ++tok) {
      const float* qs = str + (size_t)tok * NS * Dp + row_lo;
      const float* ks = qs + Dp;
      const float* ws = ks + Dp;                              // HAS_W
      const float* as = ks + (HAS_W ? 2 : 1) * Dp;            // HAS_AB
      const float* bs = as + Dp;
      const float vv = vs[tok * CB + cl];
      float sv_ = 0.f;
      if (HAS_AB) {
#pragma unroll
        for (int i = 0; i < DR; ++i) sv_ += bs[i] * S[i];
        for (int o = P >> 1; o > 0; o >>= 1) sv_ += __shfl_xor(sv_, o, 64);
      }
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < DR; ++i) {
        float upd = ks[i] * vv;
        if (HAS_AB) upd -= as[i] * sv_;
        S[i] = S[i] * (HAS_W ? ws[i] : dconst) + upd;
        acc += qs[i] * S[i];
      }
      for (int o = P >> 1; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
      if (part == 0) os[tok * CB + cl] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nt * CB; i += kScanThreads) {
      const int tok = i / CB, c = i - tok * CB;
      const int gc = blockIdx.z * CB + c;
      if (gc < E) out[(size_t)(r0 + c0 + tok) * A * E + head * E + gc] = os[i];
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DR; ++i)
      if (row_lo + i < D) sp[i] = S[i];
  }
}

}  // namespace

// rows of a column one lane keeps, and lanes per column, for a state of D rows
static void scan_shape(int D, int& DR, int& P) {
  DR = D <= 32 ? 8 : D <= 64 ? 16 : 32;
  P = 1;
  while (P * DR < D) P <<= 1;
}

int launch_state_scan(float* out, const float* q, const float* k, const float* v, const float* w, const float* a,
                      const float* b, int sq, int sk, int sv, int sw, int sa, int sb, const float* decay, float* state,
                      const int* cu_q, const int* start_pos, const int* slots, int S, int A, int D, int E,
                      hipStream_t stream) {
  if (S <= 0) return 0;
  int DR, P;
  scan_shape(D, DR, P);
  if (P > 8 || D < 1 || E < 1) return -1;
  const bool has_w = w != nullptr, has_ab = a != nullptr && b != nullptr;
  if (!has_w && decay == nullptr) return -2;
  const int NS = 2 + (has_w ? 1 : 0) + (has_ab ? 2 : 0);
  const int CB = kScanThreads / P, Dp = P * DR;
  const size_t per_tok = sizeof(float) * ((size_t)NS * Dp + 2 * CB);
  int TT = (int)((40 * 1024) / per_tok);
  TT = TT < 1 ? 1 : TT > 32 ? 32 : TT;
  const size_t shm = per_tok * TT;
  dim3 grid(S, A, (E + CB - 1) / CB);
#define RT_SCAN(DRV, HW, HAB)                                                                                          \
  do {                                                                                                                 \
    auto kern = state_scan_kernel<DRV, HW, HAB>;                                                                       \
    if (shm > 48 * 1024 &&                                                                                             \
        hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm) != hipSuccess)    \
      return -3;                                                                                                       \
    kern<<<grid, kScanThreads, shm, stream>>>(out, q, k, v, w, a, b, sq, sk, sv, sw, sa, sb, decay, state, cu_q,       \
                                              start_pos, slots, A, D, E, P, TT);                                       \
  } while (0)
#define RT_SCAN_DR(HW, HAB)                                                                                            \
  do {                                                                                                                 \
    if (DR == 8) RT_SCAN(8, HW, HAB); else if (DR == 16) RT_SCAN(16, HW, HAB); else RT_SCAN(32, HW, HAB);              \
  } while (0)
  if (has_w && has_ab) RT_SCAN_DR(true, true);
  else if (!has_w && !has_ab) RT_SCAN_DR(false, false);
  else if (has_w) RT_SCAN_DR(true, false);
  else RT_SCAN_DR(false, true);
#undef RT_SCAN_DR
#undef RT_SCAN
  return 0;
}
