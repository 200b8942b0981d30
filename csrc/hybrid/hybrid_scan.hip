// C5: matrix-state recurrence, fp32 throughout. Per sequence and head a D x E state S:
//
//   s = b_t^T S ;  S <- diag(w_t) S - a_t s^T + k_t v_t^T ;  o_t = S^T q_t
//
// (w: a stream per key channel, or one constant per head; a / b: optional removal streams.) This
// covers a constant-decay linear attention (no a / b), a generalized delta rule (a = rate * unit
// key, b = unit key) and a gated delta rule (w = g, a = g beta k, b = k, k <- beta k).
//
// The token loop is a dependent chain, so its length per token is what counts. The columns of S
// are independent; a lane owns DR rows of ONE column in registers, the P = D / DR lanes of a
// column are adjacent lanes of one DPP row (P <= 16) and add their partial dot products with
// log2(P) DPP adds (quad permutes, half-row and row mirrors: no LDS crossbar). For D = 64 that is
// 4 rows per lane: about 20 FMAs and 8 DPP adds per token. One workgroup of 256 lanes =
// (sequence, head, 256 / P columns). Tokens are staged through LDS in chunks of 16: the next
// chunk's streams are loaded into registers (16-byte loads) while the current chunk is computed,
// the operands of the next token are read from LDS while the current one is computed (a whole chunk
// is unrolled over two operand sets), and a lane's share of q . S goes to LDS as it is: the shares
// of a column are added when the chunk's outputs are written, as whole lines. The state is
// kept column by column, [slot][head][E][D], so that a lane's rows are contiguous.
#include "../common.h"

namespace {

constexpr int kScanThreads = 256;
constexpr int kTT = 16;           // tokens per staged chunk

template <int CTRL>
RT_DEVICE float dpp_add(float v) {
  const int x = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true);
  return v + __int_as_float(x);
}
// sum over the P adjacent lanes of a column (P a power of two <= 16, groups aligned to P)
RT_DEVICE float group_sum(float v, int P) {
  if (P >= 2) v = dpp_add<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  if (P >= 4) v = dpp_add<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  if (P >= 8) v = dpp_add<0x141>(v);     // row_half_mirror (quads are uniform by now)
  if (P >= 16) v = dpp_add<0x140>(v);    // row_mirror (half rows are uniform by now)
  return v;
}

// four consecutive entries r .. r + 3 of a row of D floats (zeros from D on)
RT_DEVICE float4 load4(const float* __restrict__ row, int r, int D, bool vec) {
  if (vec && r + 3 < D) return *reinterpret_cast<const float4*>(row + r);
  float4 o;
  o.x = r < D ? row[r] : 0.f;
  o.y = r + 1 < D ? row[r + 1] : 0.f;
  o.z = r + 2 < D ? row[r + 2] : 0.f;
  o.w = r + 3 < D ? row[r + 3] : 0.f;
  return o;
}

// UNROLL: whole chunks run unrolled (prompts); without it the code is a fraction of the size, which is
// what a launch over single rows (a decode step, cold instruction cache) is timed by
template <int DR, bool HAS_W, bool HAS_AB, bool UNROLL>
__global__ void __launch_bounds__(kScanThreads) state_scan_kernel(
    float* __restrict__ out, const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ w, const float* __restrict__ a, const float* __restrict__ b, int sq, int sk, int sv, int sw,
    int sa, int sb, const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ start_pos, const int* __restrict__ slots, int A, int D, int E, int P, int lgP, int vec) {
  extern __shared__ float4 lds4[];
  constexpr int NS = 2 + (HAS_W ? 1 : 0) + (HAS_AB ? 2 : 0);
  constexpr int NL = (kTT * DR + 63) / 64;      // 16-byte loads per lane, stream and chunk (P <= 16)
  constexpr int R4 = DR / 4;
  const int seq = blockIdx.x, head = blockIdx.y;
  const int CB = kScanThreads >> lgP;           // columns of this workgroup
  const int Dp4 = (P * DR) >> 2;                // padded rows / 4 (a power of two)
  const int lgDp4 = lgP + (DR == 4 ? 0 : DR == 8 ? 1 : 2);
  const int cl = threadIdx.x >> lgP, part = threadIdx.x & (P - 1);
  const int col = blockIdx.z * CB + cl;
  const int r0 = cu_q[seq], n = cu_q[seq + 1] - r0;
  if (n <= 0) return;
  float4* str = lds4;                                             // [kTT][NS][Dp4]
  float* vs = reinterpret_cast<float*>(str + kTT * NS * Dp4);     // [kTT][CB]
  float* os = vs + kTT * CB;                                      // [kTT][256]: every lane's share of q . S
  const int row_lo = part * DR;
  const bool live = col < E;
  float S[DR];
  float* sp = state + (((size_t)slots[seq] * A + head) * E + (live ? col : 0)) * D + row_lo;
  const bool cont = start_pos[seq] > 0;
  const bool svec = (D & 3) == 0;
#pragma unroll
  for (int i4 = 0; i4 < R4; ++i4) {
    float4 t = {0.f, 0.f, 0.f, 0.f};
    if (cont && live) t = load4(sp, i4 * 4, D - row_lo, svec);
    S[i4 * 4] = t.x; S[i4 * 4 + 1] = t.y; S[i4 * 4 + 2] = t.z; S[i4 * 4 + 3] = t.w;
  }
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
  float4 pre[NS][NL];
  float prev[kTT];        // this lane's share of the chunk's value columns: kTT / P entries
  const int nv = kTT >> lgP;      // 0 when P > kTT cannot happen (P <= 16 = kTT)
  auto fetch = [&](int c0) {
    const int nt = min(kTT, n - c0);
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      const float* base = src[j] + (size_t)(r0 + c0) * strides[j] + head * D;
#pragma unroll
      for (int l = 0; l < NL; ++l) {
        const int i = threadIdx.x + l * kScanThreads;
        const int tok = i >> lgDp4, r4 = i & (Dp4 - 1);
        float4 t = {0.f, 0.f, 0.f, 0.f};
        if (tok < nt) t = load4(base + (size_t)tok * strides[j], r4 * 4, D, vec != 0);
        pre[j][l] = t;
      }
    }
#pragma unroll
    for (int l = 0; l < kTT; ++l) {
      if (l < nv) {
        const int i = threadIdx.x + l * kScanThreads;
        const int tok = i / CB, c = i - tok * CB;
        const int gc = blockIdx.z * CB + c;
        prev[l] = (tok < nt && gc < E) ? v[(size_t)(r0 + c0 + tok) * sv + head * E + gc] : 0.f;
      }
    }
  };
  fetch(0);
  for (int c0 = 0; c0 < n; c0 += kTT) {
    const int nt = min(kTT, n - c0);
    __syncthreads();      // the previous chunk's readers are done
#pragma unroll
    for (int j = 0; j < NS; ++j) {
#pragma unroll
      for (int l = 0; l < NL; ++l) {
        const int i = threadIdx.x + l * kScanThreads;
        const int tok = i >> lgDp4, r4 = i & (Dp4 - 1);
        if (tok < kTT) str[(tok * NS + j) * Dp4 + r4] = pre[j][l];
      }
    }
#pragma unroll
    for (int l = 0; l < kTT; ++l)
      if (l < nv) vs[threadIdx.x + l * kScanThreads] = prev[l];
    __syncthreads();
    if (c0 + kTT < n) fetch(c0 + kTT);      // in flight while this chunk is computed
    // One token: s = b . S (summed over the column's lanes, the only cross-lane step on the chain),
    // the update, and this lane's share of q . S, which goes to LDS as it is: the shares of a
    // column are added when the chunk's outputs are written, not inside the token loop.
    auto step = [&](int tok, const float4* tq, const float4* tk, const float4* tw, const float4* ta, const float4* tb,
                    float vv) {
      float sv_ = 0.f;
      if (HAS_AB) {
#pragma unroll
        for (int i4 = 0; i4 < R4; ++i4) {
          const float4 bb = tb[i4];
          sv_ += bb.x * S[i4 * 4] + bb.y * S[i4 * 4 + 1] + bb.z * S[i4 * 4 + 2] + bb.w * S[i4 * 4 + 3];
        }
        sv_ = group_sum(sv_, P);
      }
      float acc = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < R4; ++i4) {
        const float4 kk = tk[i4], qq = tq[i4];
        float u0 = kk.x * vv, u1 = kk.y * vv, u2 = kk.z * vv, u3 = kk.w * vv;
        if (HAS_AB) {
          const float4 aa = ta[i4];
          u0 -= aa.x * sv_; u1 -= aa.y * sv_; u2 -= aa.z * sv_; u3 -= aa.w * sv_;
        }
        float d0 = dconst, d1 = dconst, d2 = dconst, d3 = dconst;
        if (HAS_W) {
          const float4 ww = tw[i4];
          d0 = ww.x; d1 = ww.y; d2 = ww.z; d3 = ww.w;
        }
        S[i4 * 4] = S[i4 * 4] * d0 + u0;
        S[i4 * 4 + 1] = S[i4 * 4 + 1] * d1 + u1;
        S[i4 * 4 + 2] = S[i4 * 4 + 2] * d2 + u2;
        S[i4 * 4 + 3] = S[i4 * 4 + 3] * d3 + u3;
        acc += qq.x * S[i4 * 4] + qq.y * S[i4 * 4 + 1] + qq.z * S[i4 * 4 + 2] + qq.w * S[i4 * 4 + 3];
      }
      os[tok * kScanThreads + threadIdx.x] = acc;
    };
    auto read_tok = [&](int tok, float4* tq, float4* tk, float4* tw, float4* ta, float4* tb, float& tv) {
      const float4* qs = str + (tok * NS) * Dp4 + part * R4;
      const float4* ks = qs + Dp4;
      const float4* ws = ks + Dp4;                              // HAS_W
      const float4* as = ks + (HAS_W ? 2 : 1) * Dp4;            // HAS_AB
      const float4* bs = as + Dp4;
#pragma unroll
      for (int i4 = 0; i4 < R4; ++i4) {
        tq[i4] = qs[i4];
        tk[i4] = ks[i4];
        if (HAS_W) tw[i4] = ws[i4];
        if (HAS_AB) {
          ta[i4] = as[i4];
          tb[i4] = bs[i4];
        }
      }
      tv = vs[tok * CB + cl];
    };
    if (UNROLL && nt == kTT) {
      // a whole chunk: unrolled, two operand sets in turn, so the operands of token tok + 1 are
      // read from LDS while token tok is computed and nothing is copied
      float4 oq[2][R4], ok[2][R4], ow[2][R4], oa[2][R4], ob[2][R4];
      float ov[2];
      read_tok(0, oq[0], ok[0], ow[0], oa[0], ob[0], ov[0]);
#pragma unroll
      for (int tok = 0; tok < kTT; ++tok) {
        const int c = tok & 1, nx = c ^ 1;
        if (tok + 1 < kTT) read_tok(tok + 1, oq[nx], ok[nx], ow[nx], oa[nx], ob[nx], ov[nx]);
        step(tok, oq[c], ok[c], ow[c], oa[c], ob[c], ov[c]);
      }
    } else {
      float4 tq[R4], tk[R4], tw[R4], ta[R4], tb[R4];
      float tv;
      for (int tok = 0; tok < nt; ++tok) {
        read_tok(tok, tq, tk, tw, ta, tb, tv);
        step(tok, tq, tk, tw, ta, tb, tv);
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nt * CB; i += kScanThreads) {
      const int tok = i / CB, c = i - tok * CB;
      const int gc = blockIdx.z * CB + c;
      const float* sh = os + tok * kScanThreads + c * P;      // the column's P shares
      float o = 0.f;
      for (int j = 0; j < P; ++j) o += sh[j];
      if (gc < E) out[(size_t)(r0 + c0 + tok) * A * E + head * E + gc] = o;
    }
  }
  if (live) {
    if (svec && row_lo + DR <= D) {
#pragma unroll
      for (int i4 = 0; i4 < R4; ++i4) {
        float4 t = {S[i4 * 4], S[i4 * 4 + 1], S[i4 * 4 + 2], S[i4 * 4 + 3]};
        *reinterpret_cast<float4*>(sp + i4 * 4) = t;
      }
    } else {
#pragma unroll
      for (int i = 0; i < DR; ++i)
        if (row_lo + i < D) sp[i] = S[i];
    }
  }
}

}  // namespace

// rows of a column one lane keeps, and lanes per column (a power of two <= 16), for D state rows
static void scan_shape(int D, int& DR, int& P, int& lgP) {
  DR = D <= 64 ? 4 : D <= 128 ? 8 : 16;
  P = 1;
  lgP = 0;
  while (P * DR < D) {
    P <<= 1;
    ++lgP;
  }
}

int launch_state_scan(float* out, const float* q, const float* k, const float* v, const float* w, const float* a,
                      const float* b, int sq, int sk, int sv, int sw, int sa, int sb, const float* decay, float* state,
                      const int* cu_q, const int* start_pos, const int* slots, int S, int T, int A, int D, int E,
                      hipStream_t stream) {
  if (S <= 0) return 0;
  const bool unroll = T > 2 * S;      // rows per span on average: single rows take the small kernel
  int DR, P, lgP;
  scan_shape(D, DR, P, lgP);
  if (P > 16 || D < 1 || E < 1) return -1;
  const bool has_w = w != nullptr, has_ab = a != nullptr && b != nullptr;
  if (!has_w && decay == nullptr) return -2;
  if (!has_w && has_ab) return -4;
  const int NS = 2 + (has_w ? 1 : 0) + (has_ab ? 2 : 0);
  const int CB = kScanThreads / P, Dp = P * DR;
  // 16-byte loads of the streams: every row start and the head offset on a 16-byte boundary
  auto al = [&](const float* p, int st) { return p == nullptr || ((reinterpret_cast<uintptr_t>(p) & 15) == 0 && (st & 3) == 0); };
  const int vec = (D & 3) == 0 && al(q, sq) && al(k, sk) && al(w, sw) && al(a, sa) && al(b, sb) ? 1 : 0;
  const size_t shm = sizeof(float) * (size_t)kTT * ((size_t)NS * Dp + CB + kScanThreads);
  dim3 grid(S, A, (E + CB - 1) / CB);
#define RT_SCAN(DRV, HW, HAB)                                                                                          \
  do {                                                                                                                 \
    if (unroll) RT_SCAN_U(DRV, HW, HAB, true); else RT_SCAN_U(DRV, HW, HAB, false);                                    \
  } while (0)
#define RT_SCAN_U(DRV, HW, HAB, UN)                                                                                    \
  do {                                                                                                                 \
    auto kern = state_scan_kernel<DRV, HW, HAB, UN>;                                                                   \
    if (shm > 48 * 1024 &&                                                                                             \
        hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm) != hipSuccess)    \
      return -3;                                                                                                       \
    kern<<<grid, kScanThreads, shm, stream>>>(out, q, k, v, w, a, b, sq, sk, sv, sw, sa, sb, decay, state, cu_q,       \
                                              start_pos, slots, A, D, E, P, lgP, vec);                                 \
  } while (0)
#define RT_SCAN_DR(HW, HAB)                                                                                            \
  do {                                                                                                                 \
    if (DR == 4) RT_SCAN(4, HW, HAB); else if (DR == 8) RT_SCAN(8, HW, HAB); else RT_SCAN(16, HW, HAB);                \
  } while (0)
  if (has_w && has_ab) RT_SCAN_DR(true, true);
  else if (!has_w) RT_SCAN_DR(false, false);
  else RT_SCAN_DR(true, false);
#undef RT_SCAN_DR
#undef RT_SCAN
#undef RT_SCAN_U
  return 0;
}
