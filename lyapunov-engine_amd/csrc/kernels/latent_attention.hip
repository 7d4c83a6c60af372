// Attention over a paged cache of latents on the matrix cores, for a prompt's
// rows and for single decoded tokens alike.
//
// Every token keeps one row of DK = KV + RD values in its page slot: the
// key/value latent (KV values) and the rotated key part shared by all heads
// (RD values).  Queries arrive already carried into the latent space
// (qa [rows, heads, DK]), so all heads of a token read the same key rows, and a
// key row's first KV values are its value as well: one load of a key tile into
// LDS serves scores and sums for every head.  KV and RD are compile-time
// constants (multiples of 16); the library is built per pair on first use.
//
// Work: the (token, head) pairs of a request, flattened token by token, are cut
// into groups of 64 rows; a workgroup of four waves takes one group (16 rows a
// wave) and one partition of the keys.  All four waves load a tile of keys into
// LDS together, row by row for the scores and transposed for the sums; each then
// computes, per 32 keys in bfloat16 (16x16x32 instructions) and per 16 in float,
//     S^T = K Q^T          (keys x rows; the accumulator leaves every lane with one
//                           row's scores for four keys, which is the operand layout
//                           of the next product, so the weights never leave registers)
//     O^T += V^T P^T       (latent dimensions x rows; a lane's accumulators all belong
//                           to its one row, so rescaling needs no exchange)
// with the softmax in 32-bit between them (running maximum and sum per row).
// With one partition the kernel finishes the softmax itself, the sink included;
// with several it leaves (maximum, sum, unnormalised sums) per partition for
// latent_combine_kernel.  The order of additions for a row depends on the
// partition size and on the row's place in its tile only through rounding.
#include <algorithm>

#include "common.h"

#ifndef LYP_LATENT_KV
#error "LYP_LATENT_KV and LYP_LATENT_RD must be defined"
#endif

namespace lyp {

constexpr int KV = LYP_LATENT_KV;
constexpr int RD = LYP_LATENT_RD;
constexpr int DK = KV + RD;
static_assert(KV % 16 == 0 && RD % 16 == 0 && KV > 0, "latent sizes in multiples of 16");
constexpr int kRowsPerGroup = 64;

// LDS of a workgroup: a tile of keys row by row (Kr, for the scores) and the same tile's first KV
// columns transposed (Vt[dimension][key], for the sums), so that both products read their operand
// along the dimension they add over.  Vt's groups of four keys are stored at swizzled places
// (swizzle below), which keeps reads and staging writes off each other's banks.
template <typename T>
struct Tile {
  static constexpr int kPad = 16 / sizeof(T);
  static constexpr int kLdK = DK + kPad;
  static constexpr size_t bytes(int keys) { return (static_cast<size_t>(keys) * kLdK + static_cast<size_t>(KV) * keys) * sizeof(T); }
  // keys staged per round: as many as 80 KiB of LDS hold, 64 or 32
  static constexpr int kKeys = bytes(64) <= 80 * 1024 ? 64 : 32;
  static constexpr size_t kBytes = bytes(kKeys);
  static_assert(kBytes <= 160 * 1024, "a tile of 32 keys must fit the LDS");
};

// Where row d of Vt keeps its groups of four keys: group g stands at g ^ swizzle(d).  Both the
// sums' reads (16 neighbouring rows, one group) and the staging writes (rows 4 i + e of 16
// neighbouring i, one group) then fall on 16 different places.
template <int NQ>
__device__ __forceinline__ int swizzle(int d) {
  return (d % NQ) ^ ((d / NQ) & 3);
}

template <typename T>
__global__ __launch_bounds__(256, KV <= 256 ? 2 : 1) void latent_attn_kernel(
    const T* __restrict__ qa, const T* __restrict__ pages, const int32_t* __restrict__ block_tables, int table_width,
    int page_size, const int32_t* __restrict__ q_start, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ ctx_len, int B, const float* __restrict__ sink, float scale, T* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, int H, int n_parts, int part_keys, int page_shift) {
  using MW = Mma16Wide<T>;                 // 16 x 16 tile over KCH values of the inner dimension
  using WFrag = typename MW::Frag;
  using M4 = Mma16<T>;                     // the same over 16 values (four a lane)
  using Frag = typename M4::Frag;
  constexpr int KE = MW::kElems;           // inner-dimension values a lane holds: 8 (bfloat16) or 4 (float)
  constexpr int KCH = 4 * KE;              // inner-dimension values per instruction: 32 or 16
  constexpr int NS = KE / 4;               // 16-key subtiles per step of the sums: 2 or 1
  constexpr int LDK = Tile<T>::kLdK;
  constexpr int KT = Tile<T>::kKeys;
  constexpr int NQ = KT / 4;               // groups of four keys in a tile
  constexpr int NCW = DK / KCH;            // full chunks of the key dimension
  constexpr bool TAIL = DK % KCH != 0;     // 16 more values (bfloat16 with DK = 32 n + 16)
  constexpr int NV = KV / 16;              // chunks of the value dimension
  constexpr int DQ = DK / 4;               // groups of four dimensions in a key row
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* Kr = reinterpret_cast<T*>(smem_raw);
  T* Vt = Kr + KT * LDK;

  // which request and which group of its rows
  int rem = blockIdx.x, b = 0, rows_b = 0;
  for (; b < B; ++b) {
    rows_b = (q_start[b + 1] - q_start[b]) * H;
    const int groups = (rows_b + kRowsPerGroup - 1) / kRowsPerGroup;
    if (rem < groups) break;
    rem -= groups;
  }
  if (b == B) return;
  const int part = blockIdx.y;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int col = lane % 16, grp = lane / 16;
  const int q0 = q_start[b];
  const bool live = ctx_len[b] > 0;
  const int row0 = rem * kRowsPerGroup;

  // this lane's row: flattened (token, head) of the request
  const int r = row0 + wave * 16 + col;
  const bool exists = r < rows_b;
  const bool valid = live && exists;
  const int tok = q0 + (exists ? r / H : 0), head = exists ? r % H : 0;
  const int limit = valid ? positions[tok] + 1 : 0;   // keys [0, limit) are seen
  const size_t grow = static_cast<size_t>(tok) * H + head;

  // keys this workgroup walks: its partition, up to what its last row sees
  const int last_row = min(row0 + kRowsPerGroup, rows_b) - 1;
  const int group_end = live ? positions[q0 + last_row / H] + 1 : 0;
  const int k_begin = part * part_keys;
  const int k_end = min(group_end, k_begin + part_keys);
  const int wave_last = min(row0 + wave * 16 + 16, rows_b) - 1;
  const int wave_end = (live && wave_last >= row0 + wave * 16) ? positions[q0 + wave_last / H] + 1 : 0;

  WFrag qf[NCW > 0 ? NCW : 1];
  Frag qtail;
  {
    const T* qrow = qa + grow * DK;
#pragma unroll
    for (int c = 0; c < NCW; ++c) {
      if (valid) qf[c] = *reinterpret_cast<const WFrag*>(qrow + c * KCH + KE * grp);
      else
#pragma unroll
        for (int e = 0; e < KE; ++e) qf[c][e] = from_f32<T>(0.f);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) qtail[e] = from_f32<T>(0.f);
    if constexpr (TAIL)
      if (valid) qtail = *reinterpret_cast<const Frag*>(qrow + NCW * KCH + 4 * grp);
  }
  f32x4 o[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) o[v] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = LYP_NEG_INF, l = 0.f;

  const int32_t* table = block_tables + static_cast<size_t>(b) * table_width;
  // Where a tile's keys lie in the pages (row numbers, -1 for none) is worked out a tile ahead by
  // the first KT threads and kept in LDS, so that the loads of the keys themselves depend on no
  // other load; a thread asks for all of its share of a tile at once (groups of four keys x four
  // dimensions: four loads, four row writes, four transposed writes each).
  __shared__ int rowidx[2][KT];
  auto locate = [&](int k0, int buf) {
    if (tid < KT) {
      const int key = k0 + tid;
      int row = -1;
      if (key < k_end) {
        const int page = page_shift >= 0 ? table[key >> page_shift] : table[key / page_size];
        const int slot = page_shift >= 0 ? key & (page_size - 1) : key % page_size;
        if (page >= 0) row = page * page_size + slot;
      }
      rowidx[buf][tid] = row;
    }
  };
  constexpr int UNITS = NQ * DQ;
  constexpr int TURNS = (UNITS + 255) / 256;
  locate(k_begin, 0);
  int buf = 0;
  for (int k0 = k_begin; k0 < k_end; k0 += KT, buf ^= 1) {
    __syncthreads();   // the tile before this one has been used by every wave; rowidx[buf] is written
    // in rounds of up to three turns: the loads of a round are all asked for before the first is used
    constexpr int ROUND = 3;
#pragma unroll
    for (int t0 = 0; t0 < TURNS; t0 += ROUND) {
      Frag stage[ROUND][4];
#pragma unroll
      for (int t = 0; t < ROUND; ++t) {
        const int idx = tid + (t0 + t) * 256;
        const int kq = idx / DQ, dq = idx % DQ;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
          for (int e = 0; e < 4; ++e) stage[t][i][e] = from_f32<T>(0.f);
          if (t0 + t < TURNS && idx < UNITS) {
            const int row = rowidx[buf][4 * kq + i];
            if (row >= 0)
              stage[t][i] = *reinterpret_cast<const Frag*>(pages + static_cast<size_t>(row) * DK + 4 * dq);
          }
        }
      }
      if (t0 == 0 && k0 + KT < k_end) locate(k0 + KT, buf ^ 1);
#pragma unroll
      for (int t = 0; t < ROUND; ++t) {
        const int idx = tid + (t0 + t) * 256;
        if (t0 + t < TURNS && idx < UNITS) {
          const int kq = idx / DQ, dq = idx % DQ;
#pragma unroll
          for (int i = 0; i < 4; ++i) *reinterpret_cast<Frag*>(Kr + (4 * kq + i) * LDK + 4 * dq) = stage[t][i];
          if (4 * dq < KV) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int d = 4 * dq + e;
              Frag tr;
#pragma unroll
              for (int i = 0; i < 4; ++i) tr[i] = stage[t][i][e];
              *reinterpret_cast<Frag*>(Vt + d * KT + 4 * (kq ^ swizzle<NQ>(d))) = tr;
            }
          }
        }
      }
    }
    __syncthreads();
    const int tile_end = min(KT, k_end - k0);
    for (int kk = 0; kk < tile_end; kk += 16 * NS) {
      if (k0 + kk >= wave_end) break;   // nothing further is seen by this wave's rows
      f32x4 s[NS];
      float tmax = LYP_NEG_INF;
#pragma unroll
      for (int u = 0; u < NS; ++u) {
        s[u] = f32x4{0.f, 0.f, 0.f, 0.f};
        f32x4 s2 = f32x4{0.f, 0.f, 0.f, 0.f};   // odd chunks: two chains of dependent products instead of one
        const T* krow = Kr + (kk + 16 * u + col) * LDK;
#pragma unroll
        for (int c = 0; c < NCW; ++c) {
          const WFrag kf = *reinterpret_cast<const WFrag*>(krow + c * KCH + KE * grp);
          if (c % 2 == 0) s[u] = MW::mma(kf, qf[c], s[u]);
          else s2 = MW::mma(kf, qf[c], s2);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) s[u][e] += s2[e];
        if constexpr (TAIL) {   // the last 16 values in a product of their own, added afterwards
          const f32x4 t = M4::mma(*reinterpret_cast<const Frag*>(krow + NCW * KCH + 4 * grp), qtail,
                                  f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
          for (int e = 0; e < 4; ++e) s[u][e] += t[e];
        }
        // s[u][e]: score of key k0 + kk + 16 u + 4 grp + e for row `col`
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = k0 + kk + 16 * u + 4 * grp + e;
          s[u][e] = key < limit ? s[u][e] * scale : LYP_NEG_INF;
          tmax = fmaxf(tmax, s[u][e]);
        }
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      const float m_new = fmaxf(m, tmax);
      float alpha = 1.f, psum = 0.f;
      WFrag pf;
      if (m_new > LYP_NEG_INF) {
        alpha = expf(m - m_new);   // m = -inf: 0
#pragma unroll
        for (int u = 0; u < NS; ++u)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float p = expf(s[u][e] - m_new);
            psum += p;
            pf[4 * u + e] = from_f32<T>(p);
          }
      } else {
#pragma unroll
        for (int e = 0; e < KE; ++e) pf[e] = from_f32<T>(0.f);
      }
      psum += __shfl_xor(psum, 16, kWave);
      psum += __shfl_xor(psum, 32, kWave);
      l = l * alpha + psum;
      m = m_new;
      const int quad = kk / 4 + grp;
      const bool rescale = __any(alpha != 1.f);   // the sums are rescaled only when some row's maximum grew
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const int d = v * 16 + col;
        const T* vrow = Vt + d * KT;
        WFrag vf;
#pragma unroll
        for (int u = 0; u < NS; ++u) {
          const Frag piece = *reinterpret_cast<const Frag*>(vrow + 4 * ((quad + 4 * u) ^ swizzle<NQ>(d)));
#pragma unroll
          for (int e = 0; e < 4; ++e) vf[4 * u + e] = piece[e];
        }
        if (rescale)
#pragma unroll
          for (int e = 0; e < 4; ++e) o[v][e] *= alpha;
        o[v] = MW::mma(vf, pf, o[v]);
      }
    }
  }
  if (!exists) return;   // no such row (no barrier follows)
  // o[v][e]: latent dimension 16 v + 4 grp + e of row `col`
  if (n_parts == 1) {
    T* orow = out + grow * KV;
    float inv = 0.f, w = 0.f;
    if (valid) {
      const float sk = sink[head];
      const float mx = fmaxf(m, sk);
      w = expf(m - mx);
      inv = 1.0f / (l * w + expf(sk - mx));
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      Frag res;
#pragma unroll
      for (int e = 0; e < 4; ++e) res[e] = from_f32<T>(valid ? o[v][e] * w * inv : 0.f);
      *reinterpret_cast<Frag*>(orow + v * 16 + 4 * grp) = res;
    }
  } else {
    float* prow = part_o + (grow * n_parts + part) * KV;
#pragma unroll
    for (int v = 0; v < NV; ++v) *reinterpret_cast<f32x4*>(prow + v * 16 + 4 * grp) = o[v];
    if (grp == 0) {
      part_ml[(grow * n_parts + part) * 2] = valid ? m : LYP_NEG_INF;
      part_ml[(grow * n_parts + part) * 2 + 1] = valid ? l : 0.f;
    }
  }
}

// One wave per (token, head) row: merges the partitions' results and the sink.
template <typename T>
__global__ __launch_bounds__(256) void latent_combine_kernel(const float* __restrict__ part_o,
                                                            const float* __restrict__ part_ml,
                                                            const float* __restrict__ sink, T* __restrict__ out,
                                                            int H, int n_parts) {
  __shared__ float weight[256];   // at most 256 partitions (lyp_latent_attn checks)
  const size_t row = blockIdx.x;
  const int head = static_cast<int>(row % H);
  const float sk = sink[head];
  __shared__ float denom_s;
  // the first wave, a lane a partition: maxima, weights and the denominator (partitions added in
  // lane order); then a thread a dimension
  if (threadIdx.x < kWave) {
    float mx = sk;
    for (int p = threadIdx.x; p < n_parts; p += kWave) mx = fmaxf(mx, part_ml[(row * n_parts + p) * 2]);
    mx = wave_max(mx);
    float part = 0.f;
    for (int p = threadIdx.x; p < n_parts; p += kWave) {
      const float mp = part_ml[(row * n_parts + p) * 2];
      const float w = mp > LYP_NEG_INF ? expf(mp - mx) : 0.f;
      weight[p] = w;
      part += part_ml[(row * n_parts + p) * 2 + 1] * w;
    }
    part = wave_sum(part);
    if (threadIdx.x == 0) denom_s = part + expf(sk - mx);
  }
  __syncthreads();
  const float inv = 1.0f / denom_s;
  for (int d = threadIdx.x; d < KV; d += blockDim.x) {
    float acc = 0.f;
#pragma unroll 4
    for (int p = 0; p < n_parts; ++p) acc += part_o[(row * n_parts + p) * KV + d] * weight[p];
    out[row * KV + d] = from_f32<T>(acc * inv);
  }
}

// For steps of few rows: the merge pass and the per-head value projection in one kernel.  One
// workgroup per (token, head) row: the row of KV latent sums (merged from the partitions as
// latent_combine_kernel does, or read from `mixed` when the keys were in one partition; rounded to
// the activations' type either way, as the two-kernel path leaves it), then out[row, v] =
// sum_r row[r] * w[head, v, r], four threads an output.
template <typename T>
__global__ __launch_bounds__(256) void latent_heads_out_kernel(const float* __restrict__ part_o,
                                                               const float* __restrict__ part_ml,
                                                               const float* __restrict__ sink,
                                                               const T* __restrict__ mixed, const T* __restrict__ w,
                                                               T* __restrict__ out, int H, int n_parts, int vdim) {
  __shared__ float weight[256];
  __shared__ float denom_s;
  __shared__ float rowv[KV];
  const size_t row = blockIdx.x;
  const int head = static_cast<int>(row % H);
  if (mixed) {
    for (int d = threadIdx.x; d < KV; d += blockDim.x) rowv[d] = to_f32(mixed[row * KV + d]);
  } else {
    const float sk = sink[head];
    if (threadIdx.x < kWave) {
      float mx = sk;
      for (int p = threadIdx.x; p < n_parts; p += kWave) mx = fmaxf(mx, part_ml[(row * n_parts + p) * 2]);
      mx = wave_max(mx);
      float part = 0.f;
      for (int p = threadIdx.x; p < n_parts; p += kWave) {
        const float mp = part_ml[(row * n_parts + p) * 2];
        const float wgt = mp > LYP_NEG_INF ? expf(mp - mx) : 0.f;
        weight[p] = wgt;
        part += part_ml[(row * n_parts + p) * 2 + 1] * wgt;
      }
      part = wave_sum(part);
      if (threadIdx.x == 0) denom_s = part + expf(sk - mx);
    }
    __syncthreads();
    const float inv = 1.0f / denom_s;
    for (int d = threadIdx.x; d < KV; d += blockDim.x) {
      float acc = 0.f;
#pragma unroll 4
      for (int p = 0; p < n_parts; ++p) acc += part_o[(row * n_parts + p) * KV + d] * weight[p];
      rowv[d] = to_f32(from_f32<T>(acc * inv));
    }
  }
  __syncthreads();
  // four neighbouring threads an output: each a quarter of the row's KV values, in pieces of four
  // (all of a thread's loads are independent), summed across the four by two exchanges
  using Frag = typename Mma16<T>::Frag;
  constexpr int SEG = KV / 4;
  const int seg = threadIdx.x % 4;
  const T* wh = w + static_cast<size_t>(head) * vdim * KV;
  for (int v0 = 0; v0 < vdim; v0 += 64) {
    const int v = v0 + threadIdx.x / 4;
    float acc = 0.f;
    if (v < vdim) {
      const T* wr = wh + static_cast<size_t>(v) * KV + seg * SEG;
#pragma unroll
      for (int r = 0; r < SEG; r += 4) {
        const Frag f = *reinterpret_cast<const Frag*>(wr + r);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc += rowv[seg * SEG + r + e] * to_f32(f[e]);
      }
    }
    acc += __shfl_xor(acc, 1, kWave);
    acc += __shfl_xor(acc, 2, kWave);
    if (v < vdim && seg == 0) out[row * vdim + v] = from_f32<T>(acc);
  }
}

}  // namespace lyp

using namespace lyp;

extern "C" {

int lyp_latent_kv_rank() { return KV; }
int lyp_latent_rot_dim() { return RD; }

// Keys per staged tile for a dtype (partition sizes are multiples of it).
int lyp_latent_tile_keys(int dtype) { return dtype == kF32 ? Tile<float>::kKeys : Tile<bf16_t>::kKeys; }

// Into how many partitions a launch had better cut the keys: few row groups and a long context
// want many workgroups; a prompt's many row groups want one partition.  `row_groups` is the
// grid's first dimension, max_ctx the longest context of the step.
int lyp_latent_plan(int row_groups, int max_ctx, int dtype) {
  const int tile = lyp_latent_tile_keys(dtype);
  const int want = 2 * compute_units();
  if (row_groups >= want || max_ctx <= tile) return 1;
  int parts = (want + row_groups - 1) / row_groups;
  parts = std::min(parts, (max_ctx + tile - 1) / tile);   // partitions of at least one tile
  return std::max(1, std::min(parts, 256));
}

// The merge of the partitions (or, with part_o == nullptr, the rows of `mixed` [rows, KV]) and the
// per-head projection w [H, vdim, KV] -> out [rows, vdim]; rows = tokens * H.  For steps of few rows.
int lyp_latent_heads_out(const float* part_o, const float* part_ml, const float* sink, const void* mixed,
                         const void* w, void* out, int dtype, int rows, int H, int n_parts, int vdim,
                         hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && H > 0 && vdim > 0 && n_parts >= 1 && n_parts <= 256, "latent_heads_out: bad sizes");
  LYP_REQUIRE((part_o != nullptr && part_ml != nullptr && sink != nullptr) != (mixed != nullptr),
              "latent_heads_out: either the partitions or the merged rows");
  if (rows == 0) return 0;
  if (dtype == kF32)
    latent_heads_out_kernel<float><<<rows, 256, 0, stream>>>(part_o, part_ml, sink, static_cast<const float*>(mixed),
                                                             static_cast<const float*>(w), static_cast<float*>(out), H,
                                                             n_parts, vdim);
  else if (dtype == kBF16)
    latent_heads_out_kernel<bf16_t><<<rows, 256, 0, stream>>>(part_o, part_ml, sink, static_cast<const bf16_t*>(mixed),
                                                              static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out),
                                                              H, n_parts, vdim);
  else
    LYP_REQUIRE(false, "latent_heads_out: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("latent_heads_out");
  return 0;
}

// qa [rows, H, DK], pages [pages, page_size, DK], out [rows, H, KV] of dtype; tables as in a step.
// merge == 0: with several partitions the merge pass is left to the caller (lyp_latent_heads_out).
// row_groups: an upper bound on the 64-row groups of all requests (rows * H / 64 rounded up, plus one
// per request).  n_parts > 1 needs part_o [rows * H * n_parts * KV] and part_ml [rows * H * n_parts * 2].
int lyp_latent_attn(const void* qa, const void* pages, const int32_t* block_tables, int table_width, int page_size,
                    const int32_t* q_start, const int32_t* positions, const int32_t* ctx_len, int B,
                    const float* sink, float scale, void* out, int dtype, int n_rows, int H, int row_groups,
                    int n_parts, int part_keys, float* part_o, float* part_ml, int merge, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && B > 0 && H > 0 && page_size > 0 && table_width > 0 && row_groups > 0,
              "latent_attn: bad sizes rows=%d B=%d H=%d page=%d", n_rows, B, H, page_size);
  LYP_REQUIRE(n_parts >= 1 && n_parts <= 256 && part_keys > 0, "latent_attn: %d partitions of %d keys", n_parts,
              part_keys);
  LYP_REQUIRE(part_keys % lyp_latent_tile_keys(dtype) == 0 || n_parts == 1,
              "latent_attn: partitions of %d keys are no multiple of the tile", part_keys);
  LYP_REQUIRE(n_parts == 1 || (part_o != nullptr && part_ml != nullptr), "latent_attn: partitions need a workspace");
  LYP_REQUIRE(reinterpret_cast<uintptr_t>(qa) % 16 == 0 && reinterpret_cast<uintptr_t>(pages) % 16 == 0,
              "latent_attn: operands must be 16-byte aligned");
  if (n_rows == 0) return 0;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0)
    for (page_shift = 0; (1 << page_shift) < page_size; ++page_shift) {}
  dim3 grid(row_groups, n_parts);
#define LYP_LATENT(T)                                                                                               \
  do {                                                                                                              \
    static bool attr_set = false;                                                                                   \
    if (!attr_set) {                                                                                                \
      hipFuncSetAttribute(reinterpret_cast<const void*>(latent_attn_kernel<T>),                                     \
                          hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(Tile<T>::kBytes));           \
      attr_set = true;                                                                                              \
    }                                                                                                               \
    latent_attn_kernel<T><<<grid, 256, Tile<T>::kBytes, stream>>>(                                                  \
        static_cast<const T*>(qa), static_cast<const T*>(pages), block_tables, table_width, page_size, q_start,     \
        positions, ctx_len, B, sink, scale, static_cast<T*>(out), part_o, part_ml, H, n_parts, part_keys,           \
        page_shift);                                                                                                \
    if (n_parts > 1 && merge)                                                                                       \
      latent_combine_kernel<T><<<n_rows * H, KV >= 256 ? 256 : (KV >= 128 ? 128 : 64), 0, stream>>>(                \
          part_o, part_ml, sink, static_cast<T*>(out), H, n_parts);                                                 \
  } while (0)
  if (dtype == kF32) LYP_LATENT(float);
  else if (dtype == kBF16) LYP_LATENT(bf16_t);
  else LYP_REQUIRE(false, "latent_attn: unknown dtype %d", dtype);
#undef LYP_LATENT
  LYP_LAUNCH_CHECK("latent_attn");
  return 0;
}

}  // extern "C"
