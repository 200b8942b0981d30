// H3: causal grouped-query attention over a paged cache with an optional softmax sink and a
// per-head score multiplier, for any head sizes up to 256 (fp32 FMA form; bf16 or fp32 tensors).
//
//   K cache [num_blocks, G, BS, Dk], V cache [num_blocks, G, BS, Dv], q [T, H, Dk], out [T, H * Dv]
//   (layout 1: the matrix-core kernels' cache — keys chunk-major per block, V [num_blocks, G, Dv, BS])
//   score(i, j) = q_i . k_j * scale * temp[h] - slopes[h] * (i - j), j <= position(i),
//                 and i - j < window when a window is given (tiles wholly ahead of it are skipped)
//   weight_j   = exp(s_j) / (sink + sum_j exp(s_j))        (sink: a key of score 0 without a value)
//   out       *= sigmoid(gate[row, h * Dv + col])          when a gate is given
//   with a soft cap c the scaled score becomes c * tanh(score / c) ahead of the distance term; the
//   result is multiplied by out_scale and may land in a column range of a wider buffer
//
// One workgroup of 4 waves = one work item (sequence, first row) x one key/value head x one key
// range: up to 32 (row, head) pairs, 8 per wave, that all read the same keys and values. The keys
// are walked in tiles of KT keys staged once in LDS as fp32 (K rows padded by one float so that
// lane = key reads are conflict-free). Scores: lane = key, one pass over the head dim for all the
// wave's pairs; online softmax per pair in registers (running maximum, sum); values: lane = value
// column, one pass over the tile's keys for all the wave's pairs. A pair's result depends only on
// its own keys, walked from key 0 in the same tile order whatever else is in the launch.
//
// Split launch (one row per sequence: a decode step): gridDim.z key ranges per work item, each
// writes (o, m, l) partials; gqa_combine_kernel merges them and adds the sink once.
#include "../common.h"

namespace {

using rt::DT;

constexpr int kPairs = 32;          // most (row, head) pairs per workgroup
constexpr int kWaves = 4;
constexpr float kNeg = -1e30f;

// DVL: value columns per lane (Dv <= 64 * DVL); kPW: pairs per wave (8: varlen tiles of 32 pairs;
// 2: the few pairs of a decode row, so no lane works on pairs that do not exist)
template <typename T, int DVL, int kPW>
__global__ void __launch_bounds__(256) gqa_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_tables, const int* __restrict__ cu_q, const int* __restrict__ start_pos,
    const int* __restrict__ tiles, const float* __restrict__ temp, float* __restrict__ part_o,
    float* __restrict__ part_ml, int H, int G, int Dk, int Dv, int BS, int max_blocks, int R, int KT, int hchunks,
    float scale, float sink, int window, const float* __restrict__ slopes, const T* __restrict__ gate,
    int gate_stride, int layout, float softcap, float out_scale, int out_stride, int out_off) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seq = tiles[2 * blockIdx.x], row0 = tiles[2 * blockIdx.x + 1];
  const int g = blockIdx.y / hchunks, hc = blockIdx.y - g * hchunks;
  const int group = H / G;
  const int h_lo = hc * kPairs, nh = min(group - h_lo, kPairs);   // this workgroup's heads of the group
  const int nrows = min(R, cu_q[seq + 1] - row0);
  const int P = nrows * nh;
  const int pos0 = start_pos[seq] + (row0 - cu_q[seq]);           // position of the tile's first row
  const int kend = pos0 + nrows;                                  // keys 0 .. kend - 1 are visible to the tile
  // this workgroup's key range (whole tiles of KT keys, counted from key 0; with a window the
  // tiles that end before the first row's oldest visible key are left out: every weight in them is 0)
  const int S = gridDim.z;
  const int ntile = (kend + KT - 1) / KT;
  const int t0 = window > 0 ? max(0, pos0 - window + 1) / KT : 0;
  const int per = (ntile - t0 + S - 1) / S;
  const int t_lo = t0 + blockIdx.z * per, t_hi = min(ntile, t_lo + per);

  float* qs = lds;                              // [kWaves * kPW][Dk]
  float* ks = qs + kWaves * kPW * Dk;           // [KT][Dk + 1]
  float* vs = ks + KT * (Dk + 1);               // [KT][Dv]
  float* ps = vs + KT * Dv;                     // [kWaves][kPW][64]
  const int* bt = block_tables + (size_t)seq * max_blocks;

  for (int i = threadIdx.x; i < P * Dk; i += blockDim.x) {
    const int p = i / Dk, d = i - p * Dk;
    const int r = p / nh, h = g * group + h_lo + (p - r * nh);
    qs[i] = DT<T>::load(q + ((size_t)(row0 + r) * H + h) * Dk + d);
  }
  float m[kPW], l[kPW], hs[kPW], sl[kPW], o[kPW][DVL];
  int qpos[kPW];
#pragma unroll
  for (int i = 0; i < kPW; ++i) {
    const int p = wave + kWaves * i;
    m[i] = kNeg;
    l[i] = 0.f;
    const int r = p / nh, h = g * group + h_lo + (p - r * nh);
    qpos[i] = p < P ? pos0 + r : -1;
    hs[i] = p < P ? scale * (temp ? temp[h] : 1.0f) : 0.f;
    sl[i] = p < P && slopes ? slopes[h] : 0.f;
#pragma unroll
    for (int c = 0; c < DVL; ++c) o[i][c] = 0.f;
  }

  for (int kt = t_lo; kt < t_hi; ++kt) {
    const int kb = kt * KT;
    __syncthreads();        // the previous tile's readers are done (and qs is written)
    for (int i = threadIdx.x; i < KT * Dk; i += blockDim.x) {
      const int j = i / Dk, d = i - j * Dk;
      const int key = kb + j;
      float v = 0.f;
      // layout 1: the cache of the matrix-core kernels (keys chunk-major per block, values [Dv][BS])
      if (key < kend)
        v = DT<T>::load(kc + ((size_t)bt[key / BS] * G + g) * BS * Dk +
                        (layout ? rt::kc_elem(BS, key % BS, d) : (key % BS) * Dk + d));
      ks[j * (Dk + 1) + d] = v;
    }
    for (int i = threadIdx.x; i < KT * Dv; i += blockDim.x) {
      const int j = i / Dv, d = i - j * Dv;
      const int key = kb + j;
      float v = 0.f;
      if (key < kend)
        v = DT<T>::load(vc + ((size_t)bt[key / BS] * G + g) * BS * Dv + (layout ? d * BS + key % BS : (key % BS) * Dv + d));
      vs[i] = v;
    }
    __syncthreads();
    // scores: lane = key
    float s[kPW];
#pragma unroll
    for (int i = 0; i < kPW; ++i) s[i] = 0.f;
    if (lane < KT) {
      const float* kr = ks + lane * (Dk + 1);
      for (int d = 0; d < Dk; ++d) {
        const float kv = kr[d];
#pragma unroll
        for (int i = 0; i < kPW; ++i) s[i] += qs[(wave + kWaves * i) * Dk + d] * kv;
      }
    }
    float alpha[kPW];
#pragma unroll
    for (int i = 0; i < kPW; ++i) {
      const int dist = qpos[i] - (kb + lane);
      const bool ok = lane < KT && dist >= 0 && (window <= 0 || dist < window);
      float raw = s[i] * hs[i];
      if (softcap > 0.f) raw = softcap * tanhf(raw / softcap);
      const float sc = ok ? raw - sl[i] * (float)dist : kNeg;
      const float mn = fmaxf(m[i], rt::wave_max(sc));
      const float pe = ok ? __expf(sc - mn) : 0.f;
      alpha[i] = __expf(m[i] - mn);
      l[i] = l[i] * alpha[i] + rt::wave_sum(pe);
      m[i] = mn;
      ps[(wave * kPW + i) * 64 + lane] = pe;
    }
    // values: lane = column (the wave's own ps rows: no workgroup barrier needed, the wave is in lockstep)
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int c = 0; c < DVL; ++c) {
      const int col = lane + 64 * c;
      if (col < Dv) {
        float acc[kPW];
#pragma unroll
        for (int i = 0; i < kPW; ++i) acc[i] = o[i][c] * alpha[i];
        for (int j = 0; j < KT; ++j) {
          const float v = vs[j * Dv + col];
#pragma unroll
          for (int i = 0; i < kPW; ++i) acc[i] += ps[(wave * kPW + i) * 64 + j] * v;
        }
#pragma unroll
        for (int i = 0; i < kPW; ++i) o[i][c] = acc[i];
      }
    }
  }

#pragma unroll
  for (int i = 0; i < kPW; ++i) {
    const int p = wave + kWaves * i;
    if (p >= P) continue;
    const int r = p / nh, h = g * group + h_lo + (p - r * nh);
    const size_t rh = (size_t)(row0 + r) * H + h;
    if (S == 1) {
      const float den = l[i] + sink * __expf(-m[i]);
      const float inv = den > 0.f ? 1.0f / den : 0.f;
#pragma unroll
      for (int c = 0; c < DVL; ++c) {
        const int col = lane + 64 * c;
        if (col < Dv) {
          float v = o[i][c] * inv * out_scale;
          if (gate) v *= 1.0f / (1.0f + __expf(-DT<T>::load(gate + (size_t)(row0 + r) * gate_stride + h * Dv + col)));
          DT<T>::store(out + (size_t)(row0 + r) * out_stride + out_off + h * Dv + col, v);
        }
      }
    } else {
      float* po = part_o + (rh * S + blockIdx.z) * Dv;
#pragma unroll
      for (int c = 0; c < DVL; ++c) {
        const int col = lane + 64 * c;
        if (col < Dv) po[col] = o[i][c];
      }
      if (lane == 0) {
        part_ml[(rh * S + blockIdx.z) * 2] = m[i];
        part_ml[(rh * S + blockIdx.z) * 2 + 1] = l[i];
      }
    }
  }
}

// one wave per (row, head): merge the S partials, add the sink once
template <typename T>
__global__ void __launch_bounds__(64) gqa_combine_kernel(T* __restrict__ out, const float* __restrict__ part_o,
                                                         const float* __restrict__ part_ml, int S, int Dv, float sink,
                                                         int H, const T* __restrict__ gate, int gate_stride,
                                                         float out_scale, int out_stride, int out_off) {
  const size_t rh = blockIdx.x;
  const int lane = threadIdx.x;
  float M = kNeg;
  for (int s = 0; s < S; ++s) M = fmaxf(M, part_ml[(rh * S + s) * 2]);
  float den = sink * __expf(-M);
  for (int s = 0; s < S; ++s) den += part_ml[(rh * S + s) * 2 + 1] * __expf(part_ml[(rh * S + s) * 2] - M);
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  for (int col = lane; col < Dv; col += 64) {
    float acc = 0.f;
    for (int s = 0; s < S; ++s) acc += part_o[(rh * S + s) * Dv + col] * __expf(part_ml[(rh * S + s) * 2] - M);
    float v = acc * inv * out_scale;
    if (gate) v *= 1.0f / (1.0f + __expf(-DT<T>::load(gate + (rh / H) * gate_stride + (rh % H) * Dv + col)));
    DT<T>::store(out + (rh / H) * out_stride + out_off + (rh % H) * Dv + col, v);
  }
}

size_t lds_bytes(int Dk, int Dv, int KT, int pairs = kPairs) {
  return sizeof(float) * ((size_t)pairs * Dk + (size_t)KT * (Dk + 1) + (size_t)KT * Dv + pairs * 64);
}

}  // namespace

// keys per staged tile: the largest of 64 / 32 / 16 / 8 whose LDS fits; 0 if none does
int gqa_key_tile(int Dk, int Dv) {
  for (int kt = 64; kt >= 8; kt >>= 1)
    if (lds_bytes(Dk, Dv, kt) <= 150 * 1024) return kt;
  return 0;
}

int launch_gqa_attention(void* out, const void* q, const void* kc, const void* vc, const int* block_tables,
                         const int* cu_q, const int* start_pos, const int* tiles, int n_tiles, const float* temp,
                         float* part_o, float* part_ml, int T, int H, int G, int Dk, int Dv, int BS, int max_blocks,
                         int rows, int num_splits, float scale, float sink, int window, const float* slopes,
                         const void* gate, int gate_stride, int layout, float softcap, float out_scale, int out_stride,
                         int out_off, bool bf, hipStream_t stream) {
  if (n_tiles <= 0 || T <= 0) return 0;
  const int KT = gqa_key_tile(Dk, Dv);
  if (KT == 0 || Dv > 256 || Dk > 256 || H % G) return -1;
  const int group = H / G;
  const int hchunks = (group + kPairs - 1) / kPairs;
  if (rows * (group < kPairs ? group : kPairs) > kPairs) return -2;
  // pairs per wave: 2 when a workgroup has at most 8 pairs (decode rows of up to 8 heads per group)
  const int pw = rows * (group < kPairs ? group : kPairs) <= 2 * kWaves ? 2 : 8;
  const size_t shm = lds_bytes(Dk, Dv, KT, kWaves * pw);
  dim3 grid(n_tiles, G * hchunks, num_splits);
  const int dvl = Dv <= 64 ? 1 : Dv <= 128 ? 2 : 4;
#define RT_GQA(TT, DVL)                                                                                              \
  do {                                                                                                               \
    if (pw == 2) RT_GQA2(TT, DVL, 2); else RT_GQA2(TT, DVL, 8);                                                      \
  } while (0)
#define RT_GQA2(TT, DVL, PW)                                                                                         \
  do {                                                                                                               \
    auto kern = gqa_attention_kernel<TT, DVL, PW>;                                                                    \
    if (shm > 48 * 1024 && hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,        \
                                               (int)shm) != hipSuccess)                                              \
      return -3;                                                                                                     \
    kern<<<grid, 256, shm, stream>>>((TT*)out, (const TT*)q, (const TT*)kc, (const TT*)vc, block_tables, cu_q,      \
                                     start_pos, tiles, temp, part_o, part_ml, H, G, Dk, Dv, BS, max_blocks, rows,   \
                                     KT, hchunks, scale, sink, window, slopes, (const TT*)gate, gate_stride, layout, \
                                     softcap, out_scale, out_stride, out_off);                                      \
  } while (0)
  if (bf) {
    if (dvl == 1) RT_GQA(uint16_t, 1); else if (dvl == 2) RT_GQA(uint16_t, 2); else RT_GQA(uint16_t, 4);
  } else {
    if (dvl == 1) RT_GQA(float, 1); else if (dvl == 2) RT_GQA(float, 2); else RT_GQA(float, 4);
  }
#undef RT_GQA
#undef RT_GQA2
  if (num_splits > 1) {
    if (bf) gqa_combine_kernel<uint16_t><<<T * H, 64, 0, stream>>>((uint16_t*)out, part_o, part_ml, num_splits, Dv, sink, H,
                                                                   (const uint16_t*)gate, gate_stride, out_scale,
                                                                   out_stride, out_off);
    else gqa_combine_kernel<float><<<T * H, 64, 0, stream>>>((float*)out, part_o, part_ml, num_splits, Dv, sink, H,
                                                             (const float*)gate, gate_stride, out_scale, out_stride,
                                                             out_off);
  }
  return 0;
}
