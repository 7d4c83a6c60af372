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
// LDS together; each then computes, per 16 keys,
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

template <typename T>
struct Tile {
  static constexpr int kPad = 16 / sizeof(T);
  static constexpr int kLd = DK + kPad;
  // keys staged per round: as many as 48 KiB of LDS hold, 16 to 64
  static constexpr int kKeys = (kLd * sizeof(T) * 64 <= 48 * 1024) ? 64 : ((kLd * sizeof(T) * 32 <= 48 * 1024) ? 32 : 16);
  static constexpr size_t kBytes = static_cast<size_t>(kKeys) * kLd * sizeof(T);
};

template <typename T>
__global__ __launch_bounds__(256) void latent_attn_kernel(
    const T* __restrict__ qa, const T* __restrict__ pages, const int32_t* __restrict__ block_tables, int table_width,
    int page_size, const int32_t* __restrict__ q_start, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ ctx_len, int B, const float* __restrict__ sink, float scale, T* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, int H, int n_parts, int part_keys) {
  using M = Mma16<T>;
  using Frag = typename M::Frag;
  constexpr int LD = Tile<T>::kLd;
  constexpr int KT = Tile<T>::kKeys;
  constexpr int NC = DK / 16;   // chunks of the key dimension
  constexpr int NV = KV / 16;   // chunks of the value dimension
  constexpr int VEC = 16 / sizeof(T);
  constexpr int VPR = DK / VEC;  // 16-byte vectors per key row
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* Ks = reinterpret_cast<T*>(smem_raw);

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

  Frag qf[NC];
  {
    const T* qrow = qa + grow * DK;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      if (valid) qf[c] = *reinterpret_cast<const Frag*>(qrow + c * 16 + 4 * grp);
      else
#pragma unroll
        for (int e = 0; e < 4; ++e) qf[c][e] = from_f32<T>(0.f);
    }
  }
  f32x4 o[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) o[v] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = LYP_NEG_INF, l = 0.f;

  const int32_t* table = block_tables + static_cast<size_t>(b) * table_width;
  for (int k0 = k_begin; k0 < k_end; k0 += KT) {
    __syncthreads();   // the tile before this one has been used by every wave
    for (int idx = tid; idx < KT * VPR; idx += 256) {
      const int j = idx / VPR, v = idx % VPR;
      const int key = k0 + j;
      VecT val;
#pragma unroll
      for (int e = 0; e < VEC; ++e) val[e] = from_f32<T>(0.f);
      if (key < k_end) {
        const int page = table[key / page_size];
        if (page >= 0)
          val = *reinterpret_cast<const VecT*>(pages + (static_cast<size_t>(page) * page_size + key % page_size) * DK +
                                               v * VEC);
      }
      *reinterpret_cast<VecT*>(Ks + j * LD + v * VEC) = val;
    }
    __syncthreads();
    const int tile_end = min(KT, k_end - k0);
    for (int kk = 0; kk < tile_end; kk += 16) {
      if (k0 + kk >= wave_end) break;   // nothing further is seen by this wave's rows
      f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
      const T* krow = Ks + (kk + col) * LD + 4 * grp;
#pragma unroll
      for (int c = 0; c < NC; ++c) s = M::mma(*reinterpret_cast<const Frag*>(krow + c * 16), qf[c], s);
      // s[e]: score of key k0 + kk + 4 grp + e for row `col`
      float tmax = LYP_NEG_INF;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = k0 + kk + 4 * grp + e;
        s[e] = key < limit ? s[e] * scale : LYP_NEG_INF;
        tmax = fmaxf(tmax, s[e]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      const float m_new = fmaxf(m, tmax);
      float alpha = 1.f, psum = 0.f;
      Frag pf;
      if (m_new > LYP_NEG_INF) {
        alpha = expf(m - m_new);   // m = -inf: 0
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float p = expf(s[e] - m_new);
          psum += p;
          pf[e] = from_f32<T>(p);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) pf[e] = from_f32<T>(0.f);
      }
      psum += __shfl_xor(psum, 16, kWave);
      psum += __shfl_xor(psum, 32, kWave);
      l = l * alpha + psum;
      m = m_new;
      const T* vbase = Ks + (kk + 4 * grp) * LD + col;
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        Frag vf;
#pragma unroll
        for (int e = 0; e < 4; ++e) vf[e] = vbase[e * LD + v * 16];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[v][e] *= alpha;
        o[v] = M::mma(vf, pf, o[v]);
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
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int e = 0; e < 4; ++e) orow[v * 16 + 4 * grp + e] = from_f32<T>(valid ? o[v][e] * w * inv : 0.f);
  } else {
    float* prow = part_o + (grow * n_parts + part) * KV;
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
      for (int e = 0; e < 4; ++e) prow[v * 16 + 4 * grp + e] = o[v][e];
    if (grp == 0) {
      part_ml[(grow * n_parts + part) * 2] = valid ? m : LYP_NEG_INF;
      part_ml[(grow * n_parts + part) * 2 + 1] = valid ? l : 0.f;
    }
  }
}

// One wave per (token, head) row: merges the partitions' results and the sink.
template <typename T>
__global__ __launch_bounds__(64) void latent_combine_kernel(const float* __restrict__ part_o,
                                                            const float* __restrict__ part_ml,
                                                            const float* __restrict__ sink, T* __restrict__ out,
                                                            int H, int n_parts) {
  __shared__ float weight[256];   // at most 256 partitions (lyp_latent_attn checks)
  const size_t row = blockIdx.x;
  const int head = static_cast<int>(row % H);
  const float sk = sink[head];
  // a lane a partition: maxima, weights and the denominator (partitions added in lane order)
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
  const float denom = wave_sum(part) + expf(sk - mx);
  __syncthreads();
  const float inv = 1.0f / denom;
  for (int d = threadIdx.x; d < KV; d += kWave) {
    float acc = 0.f;
    for (int p = 0; p < n_parts; ++p) acc += part_o[(row * n_parts + p) * KV + d] * weight[p];
    out[row * KV + d] = from_f32<T>(acc * inv);
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

// qa [rows, H, DK], pages [pages, page_size, DK], out [rows, H, KV] of dtype; tables as in a step.
// row_groups: an upper bound on the 64-row groups of all requests (rows * H / 64 rounded up, plus one
// per request).  n_parts > 1 needs part_o [rows * H * n_parts * KV] and part_ml [rows * H * n_parts * 2].
int lyp_latent_attn(const void* qa, const void* pages, const int32_t* block_tables, int table_width, int page_size,
                    const int32_t* q_start, const int32_t* positions, const int32_t* ctx_len, int B,
                    const float* sink, float scale, void* out, int dtype, int n_rows, int H, int row_groups,
                    int n_parts, int part_keys, float* part_o, float* part_ml, hipStream_t stream) {
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
        positions, ctx_len, B, sink, scale, static_cast<T*>(out), part_o, part_ml, H, n_parts, part_keys);          \
    if (n_parts > 1)                                                                                                \
      latent_combine_kernel<T><<<n_rows * H, 64, 0, stream>>>(part_o, part_ml, sink, static_cast<T*>(out), H,       \
                                                              n_parts);                                             \
  } while (0)
  if (dtype == kF32) LYP_LATENT(float);
  else if (dtype == kBF16) LYP_LATENT(bf16_t);
  else LYP_REQUIRE(false, "latent_attn: unknown dtype %d", dtype);
#undef LYP_LATENT
  LYP_LAUNCH_CHECK("latent_attn");
  return 0;
}

}  // extern "C"
