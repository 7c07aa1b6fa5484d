// Attention over a compressed cache: every token leaves one vector [latent | rotated key part] in its
// page slot, shared by all heads.  A head's query is brought into that space first (its unrotated part
// through the transposed key up-projection, its rotated part as it is), so that a score is one dot
// product with the cached vector and the weighted sum of cached latents is projected up to the head's
// values afterwards: the cache is read once for all heads of a row tile.
//
//   latent_prep:         RMSNorm of the latent, rotation of the shared key part and of the queries' rotated
//                        parts, cache write.
//   headwise_linear:     out[r][h] = W[h] x[r][h], a product per head with weights of its own.
//   shared_key_attention: causal softmax attention of all heads over the shared keys, values a prefix of
//                        the key vector, with an optional sink per head in the denominator and an optional window.
//
// Scores, softmax weights, norms and rotations are 32-bit whatever the cache's dtype.
#include "common.h"
#include "api.h"

#include <math.h>

namespace {

template <typename T>
__device__ __forceinline__ float load_f(const T* p) {
  if constexpr (sizeof(T) == 2) return bf16_to_f32(*p);
  else return *p;
}

template <typename T>
__device__ __forceinline__ void store_f(T* p, float v) {
  if constexpr (sizeof(T) == 2) *p = f32_to_bf16(v);
  else *p = v;
}

// ------------------------------------------------------------------------- prep

struct PrepArgs {
  const float* proj;     // [rows, ldp]: q at q_off (heads x (dim + rot)), the down projection at dkv_off (rank + rot)
  int ldp, q_off, dkv_off;
  const float* norm_w;   // [rank]
  float eps;
  const float* cos_table;   // [positions, rotary / 2]
  const float* sin_table;
  const int32_t* positions;
  const int32_t* row_seq;
  const int32_t* block_table;
  int table_stride;
  void* qa;              // [rows, ldqa] (32-bit, or bfloat16 for the matrix-core attention): head h at h * (rank + rot); the
  int ldqa, qa_is_bf16;  // rotated part goes to its last rot elements
  int heads, dim, rot, rotary, rank, page_size, write_cache;
};

// A workgroup a row.  The rotated part: elements i and i + rotary/2 (i < rotary/2) are a pair; elements from
// ``rotary`` on pass unchanged.
template <typename CT>
__global__ __launch_bounds__(256) void latent_prep_kernel(PrepArgs a, CT* __restrict__ cache, CT* __restrict__ latent_t) {
  const int row = blockIdx.x;
  const int pos = a.positions[row];
  if (pos < 0) return;
  const int lane = threadIdx.x & 63;
  const float* pr = a.proj + (size_t)row * a.ldp;
  const float* dkv = pr + a.dkv_off;
  const int half = a.rotary / 2;
  const float* ct = a.cos_table + (size_t)pos * half;
  const float* st = a.sin_table + (size_t)pos * half;
  const int width = a.rank + a.rot;
  if (a.write_cache) {
    // every wave sums the latent's squares in the same order; the lanes are joined by the butterflies of wave_sum
    float acc = 0.0f;
    for (int i = lane; i < a.rank; i += 64) acc = fmaf(dkv[i], dkv[i], acc);
    const float inv = 1.0f / sqrtf(wave_sum(acc) / (float)a.rank + a.eps);
    const int page = a.block_table[(size_t)a.row_seq[row] * a.table_stride + pos / a.page_size];
    CT* dst = cache + ((size_t)page * a.page_size + pos % a.page_size) * width;
    for (int i = threadIdx.x; i < a.rank; i += blockDim.x) store_f(dst + i, (dkv[i] * inv) * a.norm_w[i]);
    if (latent_t != nullptr) {      // the latent once more, transposed within its page: [page][element][slot]
      CT* tp = latent_t + (size_t)page * a.rank * a.page_size + pos % a.page_size;
      for (int i = threadIdx.x; i < a.rank; i += blockDim.x) store_f(tp + (size_t)i * a.page_size, (dkv[i] * inv) * a.norm_w[i]);
    }
    const float* kr = dkv + a.rank;
    for (int i = threadIdx.x; i < a.rot; i += blockDim.x) {
      float v;
      if (i < half) v = kr[i] * ct[i] - kr[i + half] * st[i];
      else if (i < a.rotary) v = kr[i] * ct[i - half] + kr[i - half] * st[i - half];
      else v = kr[i];
      store_f(dst + a.rank + i, v);
    }
  }
  const int per = a.dim + a.rot;
  for (int e = threadIdx.x; e < a.heads * a.rot; e += blockDim.x) {
    const int h = e / a.rot, i = e % a.rot;
    const float* qr = pr + a.q_off + h * per + a.dim;
    float v;
    if (i < half) v = qr[i] * ct[i] - qr[i + half] * st[i];
    else if (i < a.rotary) v = qr[i] * ct[i - half] + qr[i - half] * st[i - half];
    else v = qr[i];
    const size_t at = (size_t)row * a.ldqa + h * width + a.rank + i;
    if (a.qa_is_bf16) reinterpret_cast<bf16_t*>(a.qa)[at] = f32_to_bf16(v);
    else reinterpret_cast<float*>(a.qa)[at] = v;
  }
}

// ------------------------------------------------------------------------- a product per head

// out[r][h*ohs + o] = sum_i wt[h][i][o] * x[r][h*xhs + i]: the weights lie input-major, so that neighbouring threads
// (outputs) read neighbouring weights; HL_ROWS rows share every weight that is loaded.  One fused multiply-add chain
// per output, i ascending.
// A workgroup is 64 outputs by four quarters of the inner size (a wave a quarter, eight weights asked for at a time); the
// quarters' sums meet in LDS and are added in quarter order.
#define HL_ROWS 8
template <typename WT, typename OT>
__global__ __launch_bounds__(256) void headwise_linear_kernel(const float* __restrict__ x, int ldx, int xhs,
                                                              const WT* __restrict__ wt, int in, int outn,
                                                              OT* __restrict__ out, int ldo, int ohs, int rows) {
  extern __shared__ float hl_x[];      // [HL_ROWS][in], then [4][HL_ROWS][64] partial sums
  float* hl_part = hl_x + HL_ROWS * in;
  const int r0 = blockIdx.x * HL_ROWS, h = blockIdx.y;
  const int lane = threadIdx.x & 63, quarter = wave_index();
  const int o = blockIdx.z * 64 + lane;
  for (int e = threadIdx.x; e < HL_ROWS * in; e += 256) {
    const int r = e / in, i = e % in;
    hl_x[e] = (r0 + r < rows) ? x[(size_t)(r0 + r) * ldx + h * xhs + i] : 0.0f;
  }
  __syncthreads();
  float acc[HL_ROWS];
#pragma unroll
  for (int r = 0; r < HL_ROWS; ++r) acc[r] = 0.0f;
  const int per = (in + 3) / 4;
  const int i0 = quarter * per, i1 = min(in, i0 + per);
  const WT* wp = wt + (size_t)h * in * outn + min(o, outn - 1);
  for (int i = i0; i < i1; i += 8) {
    float w[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) w[u] = load_f(wp + (size_t)min(i + u, i1 - 1) * outn);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (i + u < i1) {
#pragma unroll
        for (int r = 0; r < HL_ROWS; ++r) acc[r] = fmaf(hl_x[r * in + i + u], w[u], acc[r]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < HL_ROWS; ++r) hl_part[(quarter * HL_ROWS + r) * 64 + lane] = acc[r];
  __syncthreads();
  if (quarter != 0 || o >= outn) return;
#pragma unroll
  for (int r = 0; r < HL_ROWS; ++r) {
    const float sum = ((hl_part[r * 64 + lane] + hl_part[(HL_ROWS + r) * 64 + lane]) + hl_part[(2 * HL_ROWS + r) * 64 + lane]) +
                      hl_part[(3 * HL_ROWS + r) * 64 + lane];
    if (r0 + r < rows) store_f(out + (size_t)(r0 + r) * ldo + h * ohs + o, sum);
  }
}

// ------------------------------------------------------------------------- attention over shared keys

struct SharedKeyArgs {
  const float* q;          // [rows, ldq]: head h at h * dk
  int ldq;
  const int32_t* positions;
  const int32_t* block_table;
  int table_stride;
  const int32_t* tiles;    // [num_tiles, 4] = (first row, rows, request, 0); null: tile t is row t of request t
  const float* sink;       // [heads] or null
  float* out;              // [rows, ldo]: head h at h * dv
  int ldo;
  int heads, dk, dv, page_size, window, hg, num_pages;
  float scale;
};

// A workgroup of four waves per (tile of rows, group of ``hg`` heads): 16 query vectors, four a wave (16 / hg rows a
// tile: hg = 4 for prompt portions, 16 for single tokens).  Keys come through LDS in blocks of KB as 32-bit rows;
// for the scores a lane is a key (each key element it reads serves the wave's four queries), for the weighted sum a
// lane is NVC value columns.  The running maximum starts at the sink and the denominator at 1 = e^(sink - sink): the sink is
// one more score that has no value.
template <typename CT, int KB, int NVC>
__global__ __launch_bounds__(256) void shared_key_attention_kernel(SharedKeyArgs a, const CT* __restrict__ cache) {
  extern __shared__ float lds[];
  const int dkp = (a.dk + 3) & ~3;
  const int kstride = dkp + 4;
  float* Ks = lds;                         // [KB][kstride]
  float* Qs = Ks + KB * kstride;           // [16][dkp]
  float* Ps = Qs + 16 * dkp;               // [16][KB]
  const int lane = threadIdx.x & 63, w = wave_index();
  const int t = blockIdx.x;
  int r0, nr, seq;
  if (a.tiles != nullptr) {
    r0 = a.tiles[4 * t];
    nr = a.tiles[4 * t + 1];
    seq = a.tiles[4 * t + 2];
  } else {
    r0 = t;
    nr = 1;
    seq = t;
  }
  if (nr <= 0) return;
  const int pos0 = a.positions[r0];
  if (pos0 < 0) return;
  const int pmax = pos0 + nr - 1;
  const int h0 = blockIdx.y * a.hg;

  // this wave's four query vectors
  int qrow[4], qh[4], qpos[4];
  bool qok[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int qv = 4 * w + g;
    const int rl = qv / a.hg;
    qh[g] = h0 + qv % a.hg;
    qok[g] = rl < nr && qh[g] < a.heads;
    qrow[g] = r0 + (rl < nr ? rl : 0);
    qpos[g] = qok[g] ? pos0 + rl : -1;
  }
  for (int e = threadIdx.x; e < 16 * dkp; e += 256) {
    const int qv = e / dkp, d = e % dkp;
    const int rl = qv / a.hg, h = h0 + qv % a.hg;
    Qs[e] = (rl < nr && h < a.heads && d < a.dk) ? a.q[(size_t)(r0 + rl) * a.ldq + h * a.dk + d] : 0.0f;
  }
  float m[4], l[4], acc[4][NVC];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const bool has = a.sink != nullptr && qok[g];
    m[g] = has ? a.sink[qh[g]] : -INFINITY;
    l[g] = has ? 1.0f : 0.0f;
#pragma unroll
    for (int c = 0; c < NVC; ++c) acc[g][c] = 0.0f;
  }
  const int lo_first = a.window > 0 ? max(0, pos0 - a.window + 1) : 0;
  const int32_t* table = a.block_table + (size_t)seq * a.table_stride;

  for (int kb0 = lo_first / KB * KB; kb0 <= pmax; kb0 += KB) {
    __syncthreads();
    // the block's keys, widened to 32-bit; keys beyond the tile's last position and the padding are zero
    for (int e = threadIdx.x; e < KB * dkp; e += 256) {
      const int jj = e / dkp, d = e % dkp;
      const int kj = kb0 + jj;
      float v = 0.0f;
      if (kj <= pmax && kj >= lo_first && d < a.dk) {
        int page = table[kj / a.page_size];
        page = min(max(page, 0), a.num_pages - 1);
        v = load_f(cache + ((size_t)page * a.page_size + kj % a.page_size) * a.dk + d);
      }
      Ks[jj * kstride + d] = v;
    }
    __syncthreads();
    float sc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (lane < KB) {
      const float* kr = Ks + lane * kstride;
      for (int d = 0; d < dkp; d += 4) {
        const f32x4 kv = *reinterpret_cast<const f32x4*>(kr + d);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 qv = *reinterpret_cast<const f32x4*>(Qs + (4 * w + g) * dkp + d);
          sc[g] = fmaf(kv[0], qv[0], sc[g]);
          sc[g] = fmaf(kv[1], qv[1], sc[g]);
          sc[g] = fmaf(kv[2], qv[2], sc[g]);
          sc[g] = fmaf(kv[3], qv[3], sc[g]);
        }
      }
    }
    const int kj = kb0 + lane;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int lo = a.window > 0 ? max(0, qpos[g] - a.window + 1) : 0;
      const bool valid = lane < KB && kj <= qpos[g] && kj >= lo;
      const float s = valid ? sc[g] * a.scale : -INFINITY;
      const float mn = fmaxf(m[g], wave_max(s));
      const float base = mn == -INFINITY ? 0.0f : mn;
      float p, corr;
      if constexpr (sizeof(CT) == 2) {
        p = valid ? fast_exp(s - base) : 0.0f;
        corr = m[g] == -INFINITY ? 0.0f : fast_exp(m[g] - base);
      } else {
        p = valid ? bw_expf(s - base) : 0.0f;
        corr = m[g] == -INFINITY ? 0.0f : bw_expf(m[g] - base);
      }
      l[g] = l[g] * corr + wave_sum(p);
      m[g] = mn;
#pragma unroll
      for (int c = 0; c < NVC; ++c) acc[g][c] *= corr;
      if (lane < KB) Ps[(4 * w + g) * KB + lane] = p;
    }
    __syncthreads();
    for (int jj = 0; jj < KB; jj += 4) {
      f32x4 p4[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) p4[g] = *reinterpret_cast<const f32x4*>(Ps + (4 * w + g) * KB + jj);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
#pragma unroll
        for (int c = 0; c < NVC; ++c) {
          const int col = lane + 64 * c;
          const float v = col < a.dv ? Ks[(jj + u) * kstride + col] : 0.0f;
#pragma unroll
          for (int g = 0; g < 4; ++g) acc[g][c] = fmaf(p4[g][u], v, acc[g][c]);
        }
      }
    }
  }
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    if (!qok[g]) continue;
    const float inv = l[g] > 0.0f ? 1.0f / l[g] : 0.0f;
#pragma unroll
    for (int c = 0; c < NVC; ++c) {
      const int col = lane + 64 * c;
      if (col < a.dv) a.out[(size_t)qrow[g] * a.ldo + qh[g] * a.dv + col] = acc[g][c] * inv;
    }
  }
}

template <typename CT, int KB>
int launch_shared_key_kb(const SharedKeyArgs& a, const CT* cache, int num_tiles, hipStream_t s) {
  const int dkp = (a.dk + 3) & ~3;
  const size_t bytes = ((size_t)KB * (dkp + 4) + 16 * dkp + 16 * KB) * sizeof(float);
  const dim3 grid(num_tiles, (a.heads + a.hg - 1) / a.hg), block(256);
  const int nvc = (a.dv + 63) / 64;
#define BW_SK_LAUNCH(N)                                                                                                  \
  do {                                                                                                                   \
    static bool attr_set = false;                                                                                        \
    if (!attr_set) {                                                                                                     \
      (void)hipFuncSetAttribute((const void*)shared_key_attention_kernel<CT, KB, N>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                          150 * 1024);                                                                                   \
      attr_set = true;                                                                                                   \
    }                                                                                                                    \
    hipLaunchKernelGGL((shared_key_attention_kernel<CT, KB, N>), grid, block, bytes, s, a, cache);                        \
  } while (0)
  if (nvc <= 1) BW_SK_LAUNCH(1);
  else if (nvc <= 2) BW_SK_LAUNCH(2);
  else if (nvc <= 4) BW_SK_LAUNCH(4);
  else if (nvc <= 8) BW_SK_LAUNCH(8);
  else return -4;
#undef BW_SK_LAUNCH
  return BW_LAUNCH_CHECK();
}

template <typename CT>
int launch_shared_key(const SharedKeyArgs& a, const CT* cache, int num_tiles, hipStream_t s) {
  const int dkp = (a.dk + 3) & ~3;
  const size_t budget = 144 * 1024;
  auto bytes = [&](int kb) { return ((size_t)kb * (dkp + 4) + 16 * dkp + 16 * kb) * sizeof(float); };
  // (blocks of 64 keys while two workgroups still fit a compute unit's LDS, else what fits)
  if (bytes(64) <= 72 * 1024) return launch_shared_key_kb<CT, 64>(a, cache, num_tiles, s);
  if (bytes(32) <= budget) return launch_shared_key_kb<CT, 32>(a, cache, num_tiles, s);
  if (bytes(16) <= budget) return launch_shared_key_kb<CT, 16>(a, cache, num_tiles, s);
  return -8;
}


// ------------------------------------------------------------------------- the same attention on the matrix cores

// bfloat16 caches whose key vectors are whole 16-byte groups.  A wave per (tile, group of heads, split of the keys): 16
// query vectors (16 / hg rows x hg heads), keys in blocks of 64.  Scores: v_mfma_f32_16x16x32_bf16 with the keys as rows
// (operand A, straight from the cache: a lane reads 8 consecutive elements of its key) and the queries as columns
// (operand B, rounded to bfloat16 once, from LDS); 32-bit sums, scaled, masked, softmax in 32-bit with a running maximum.
// The weighted sum takes the weights rounded to bfloat16 as columns and the values as rows d of a second copy of the
// latent that the cache write leaves transposed, [page][d][slot]: a lane's 8 keys are two runs of 4 consecutive slots
// (the keys of its four scores in two neighbouring sub-blocks of 16).  A lane's scores, sums and outputs all belong to
// query (lane mod 16).  With nsplit > 1 a wave takes kchunk keys and leaves (maximum, denominator, sums) for
// shared_key_combine_kernel; the sink joins where the result is finished.
struct MfmaAttnArgs {
  const bf16_t* q;         // [rows, ldq] bfloat16: head h at h * dk
  int ldq;
  const int32_t* positions;
  const int32_t* block_table;
  int table_stride;
  const int32_t* tiles;
  const float* sink;
  float* out;
  int ldo;
  float* partial;          // [tiles][heads][nsplit][dv + 2]
  int heads, dk, dv, page_size, window, hg, num_pages, nsplit, kchunk;
  float scale;
};

__device__ __forceinline__ float across_groups_max(float v) {
  float a, b;
  lane_halves<32>(v, a, b);
  v = fmaxf(a, b);
  lane_halves<16>(v, a, b);
  return fmaxf(a, b);
}

__device__ __forceinline__ float across_groups_sum(float v) {
  float a, b;
  lane_halves<32>(v, a, b);
  v = a + b;
  lane_halves<16>(v, a, b);
  return a + b;
}

template <int NDT>
__global__ __launch_bounds__(64) void shared_key_attention_mfma_kernel(MfmaAttnArgs a, const bf16_t* __restrict__ kc,
                                                                       const bf16_t* __restrict__ vt) {
  extern __shared__ bf16_t qs[];           // [16][qstride]
  const int lane = threadIdx.x, n = lane & 15, g = lane >> 4;
  const int t = blockIdx.x, h0 = blockIdx.y * a.hg, split = blockIdx.z;
  int r0, nr, seq;
  if (a.tiles != nullptr) {
    r0 = a.tiles[4 * t];
    nr = a.tiles[4 * t + 1];
    seq = a.tiles[4 * t + 2];
  } else {
    r0 = t;
    nr = 1;
    seq = t;
  }
  if (nr <= 0) return;
  const int pos0 = a.positions[r0];
  if (pos0 < 0) return;
  const int pmax = pos0 + nr - 1;
  const int rl = n / a.hg, h = h0 + n % a.hg;
  const bool qok = rl < nr && h < a.heads;
  const int qpos = qok ? pos0 + rl : -1;
  const int qlo = a.window > 0 ? max(0, qpos - a.window + 1) : 0;
  const int dkp = (a.dk + 31) & ~31, qstride = dkp + 8;
  {
    const int groups = dkp >> 3;             // 16-byte groups of a query vector (dk is a multiple of 8)
#pragma unroll 4
    for (int e = lane; e < 16 * groups; e += 64) {
      const int qn = e / groups, d = (e % groups) * 8;
      const int r2 = qn / a.hg, h2 = h0 + qn % a.hg;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (r2 < nr && h2 < a.heads && d < a.dk) v = *reinterpret_cast<const u32x4*>(a.q + (size_t)(r0 + r2) * a.ldq + h2 * a.dk + d);
      *reinterpret_cast<u32x4*>(qs + qn * qstride + d) = v;
    }
  }
  __syncthreads();

  const int lo_first = a.window > 0 ? max(0, pos0 - a.window + 1) : 0;
  int k_begin = lo_first & ~63, k_end = pmax + 1;
  if (a.nsplit > 1) {
    k_begin = max(k_begin, split * a.kchunk);
    k_end = min(k_end, (split + 1) * a.kchunk);
  }
  const int32_t* table = a.block_table + (size_t)seq * a.table_stride;
  const int ps = a.page_size, dk = a.dk, dv = a.dv;

  float m = -INFINITY, lsum = 0.0f;
  f32x4 acc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) acc[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  for (int kb0 = k_begin; kb0 < k_end; kb0 += 64) {
    const bf16_t* krow[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int kj = min(kb0 + 16 * u + n, pmax);
      const int page = min(max(table[kj / ps], 0), a.num_pages - 1);
      krow[u] = kc + ((size_t)page * ps + kj % ps) * dk;
    }
    // (where the values' runs of 4 keys lie: asked of the table together with the keys' pages)
    const bf16_t* vrun[2][2];
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const int c = min(kb0 + 32 * w + 16 * x + 4 * g, pmax & ~3);
        vrun[w][x] = vt + (size_t)min(max(table[c / ps], 0), a.num_pages - 1) * dv * ps + c % ps;
      }
    f32x4 st[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) st[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // KST steps of 32 elements at a time: their 4 KST loads are in flight together (a single token's piece of 64 keys
    // is one block, and what it waits for is memory)
    constexpr int KST = NDT <= 16 ? 10 : 6;
    for (int d1 = 8 * g; d1 < dkp; d1 += 32 * KST) {
      u32x4 kf[KST][4], qf[KST];
#pragma unroll
      for (int s4 = 0; s4 < KST; ++s4) {
        const int d0 = d1 + 32 * s4;
        qf[s4] = d0 < dkp ? *reinterpret_cast<const u32x4*>(qs + n * qstride + d0) : (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < 4; ++u) kf[s4][u] = d0 < dk ? *reinterpret_cast<const u32x4*>(krow[u] + d0) : (u32x4){0u, 0u, 0u, 0u};
      }
#pragma unroll
      for (int s4 = 0; s4 < KST; ++s4)
#pragma unroll
        for (int u = 0; u < 4; ++u)
          st[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf[s4][u]), as_bf16x8(qf[s4]), st[u], 0, 0, 0);
    }
    // this lane: query n, keys kb0 + 16u + 4g + i
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = kb0 + 16 * u + 4 * g + i;
        const bool valid = key <= qpos && key >= qlo && key < k_end;
        const float sv = valid ? st[u][i] * a.scale : -INFINITY;
        st[u][i] = sv;
        mx = fmaxf(mx, sv);
      }
    mx = across_groups_max(mx);
    const float mn = fmaxf(m, mx);
    const float base = mn == -INFINITY ? 0.0f : mn;
    const float corr = m == -INFINITY ? 0.0f : fast_exp(m - base);
    float psum = 0.0f;
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = st[u][i] == -INFINITY ? 0.0f : fast_exp(st[u][i] - base);
        st[u][i] = pv;
        psum += pv;
      }
    lsum = lsum * corr + psum;
    m = mn;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) acc[dt] *= corr;
    const bool ragged = kb0 + 63 > pmax || kb0 < lo_first;       // slots behind the last key, or before the window, may hold anything
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const u32x4 pf = {pack_bf16x2(st[2 * w][0], st[2 * w][1]), pack_bf16x2(st[2 * w][2], st[2 * w][3]),
                        pack_bf16x2(st[2 * w + 1][0], st[2 * w + 1][1]), pack_bf16x2(st[2 * w + 1][2], st[2 * w + 1][3])};
      const int key0 = kb0 + 32 * w + 4 * g, key1 = key0 + 16;
      const bf16_t* b0 = vrun[w][0];
      const bf16_t* b1 = vrun[w][1];
      uint32_t keep0[2] = {0xffffffffu, 0xffffffffu}, keep1[2] = {0xffffffffu, 0xffffffffu};
      if (ragged) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t bits = 0xffffu << (16 * (e & 1));
          if (key0 + e > pmax || key0 + e < lo_first) keep0[e >> 1] &= ~bits;
          if (key1 + e > pmax || key1 + e < lo_first) keep1[e >> 1] &= ~bits;
        }
      }
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        const int d = 16 * dt + n;
        u32x4 vf = {0u, 0u, 0u, 0u};
        if (d < dv) {
          const u32x2 x0 = *reinterpret_cast<const u32x2*>(b0 + (size_t)d * ps);
          const u32x2 x1 = *reinterpret_cast<const u32x2*>(b1 + (size_t)d * ps);
          vf = (u32x4){x0[0] & keep0[0], x0[1] & keep0[1], x1[0] & keep1[0], x1[1] & keep1[1]};
        }
        acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf), as_bf16x8(pf), acc[dt], 0, 0, 0);
      }
    }
  }
  lsum = across_groups_sum(lsum);
  if (!qok) return;
  if (a.nsplit > 1) {
    float* part = a.partial + (((size_t)t * a.heads + h) * a.nsplit + split) * (dv + 2);
    if (g == 0) {
      part[0] = m;
      part[1] = lsum;
    }
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 16 * dt + 4 * g + i;
        if (d < dv) part[2 + d] = acc[dt][i];
      }
    return;
  }
  const float sk = a.sink != nullptr ? a.sink[h] : -INFINITY;
  const float mf = fmaxf(m, sk);
  const float cm = m == -INFINITY ? 0.0f : fast_exp(m - mf);
  const float lt = lsum * cm + (sk == -INFINITY ? 0.0f : fast_exp(sk - mf));
  const float w = lt > 0.0f ? cm / lt : 0.0f;
  float* orow = a.out + (size_t)(r0 + rl) * a.ldo + h * dv;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = 16 * dt + 4 * g + i;
      if (d < dv) orow[d] = acc[dt][i] * w;
    }
}

// The splits of one (single-row tile, head) joined: the largest maximum (the sink's score among them), every split's
// denominator and sums scaled to it, in split order.
__global__ __launch_bounds__(64) void shared_key_combine_kernel(MfmaAttnArgs a) {
  const int t = blockIdx.x, h = blockIdx.y;
  const int r0 = a.tiles != nullptr ? a.tiles[4 * t] : t;
  if (a.tiles != nullptr && a.tiles[4 * t + 1] <= 0) return;
  if (a.positions[r0] < 0) return;
  const float* part = a.partial + ((size_t)t * a.heads + h) * a.nsplit * (a.dv + 2);
  const int live = min(a.nsplit, a.positions[r0] / a.kchunk + 1);      // splits beyond the row's position hold nothing
  const float sk = a.sink != nullptr ? a.sink[h] : -INFINITY;
  // lane s holds split s's maximum and denominator (at most 64 splits); the weights of the splits go through LDS
  __shared__ float wgt[64];
  const int lane = threadIdx.x;
  const float ms = lane < live ? part[(size_t)lane * (a.dv + 2)] : -INFINITY;
  const float ls = lane < live ? part[(size_t)lane * (a.dv + 2) + 1] : 0.0f;
  const float mt = fmaxf(sk, wave_max(ms));
  const float ws = ms == -INFINITY ? 0.0f : fast_exp(ms - mt);
  const float lt = wave_sum(ls * ws) + (sk == -INFINITY ? 0.0f : fast_exp(sk - mt));
  wgt[lane] = ws;
  __syncthreads();
  const float inv = lt > 0.0f ? 1.0f / lt : 0.0f;
  for (int d = lane; d < a.dv; d += 64) {
    float o = 0.0f;
    for (int s0 = 0; s0 < live; s0 += 8) {
      float pv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) pv[u] = part[(size_t)min(s0 + u, live - 1) * (a.dv + 2) + 2 + d];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < live && wgt[s0 + u] != 0.0f) o = fmaf(pv[u], wgt[s0 + u], o);
    }
    a.out[(size_t)r0 * a.ldo + h * a.dv + d] = o * inv;
  }
}

int launch_shared_key_mfma(const MfmaAttnArgs& a, const bf16_t* kc, const bf16_t* vt, int num_tiles, hipStream_t s) {
  const int dkp = (a.dk + 31) & ~31;
  const size_t bytes = (size_t)16 * (dkp + 8) * sizeof(bf16_t);
  const dim3 grid(num_tiles, (a.heads + a.hg - 1) / a.hg, a.nsplit), block(64);
  const int ndt = (a.dv + 15) / 16;
  if (ndt <= 4) hipLaunchKernelGGL(shared_key_attention_mfma_kernel<4>, grid, block, bytes, s, a, kc, vt);
  else if (ndt <= 8) hipLaunchKernelGGL(shared_key_attention_mfma_kernel<8>, grid, block, bytes, s, a, kc, vt);
  else if (ndt <= 16) hipLaunchKernelGGL(shared_key_attention_mfma_kernel<16>, grid, block, bytes, s, a, kc, vt);
  else if (ndt <= 32) hipLaunchKernelGGL(shared_key_attention_mfma_kernel<32>, grid, block, bytes, s, a, kc, vt);
  else return -4;
  if (a.nsplit > 1) hipLaunchKernelGGL(shared_key_combine_kernel, dim3(num_tiles, a.heads), dim3(64), 0, s, a);
  return BW_LAUNCH_CHECK();
}

}  // namespace

extern "C" int bw_latent_prep(const float* proj, int ldp, int q_off, int dkv_off, const float* norm_w, float eps,
                              const float* cos_table, const float* sin_table, const int32_t* positions,
                              const int32_t* row_seq, const int32_t* block_table, int table_stride, void* cache,
                              void* latent_t, int cache_is_bf16, void* qa, int qa_is_bf16, int ldqa, int rows, int heads, int dim, int rot, int rotary,
                              int rank, int page_size, int write_cache, void* stream) {
  if (rows <= 0) return 0;
  if (heads <= 0 || dim < 0 || rot < 0 || rotary < 0 || rotary > rot || (rotary & 1) || rank <= 0 || page_size <= 0) return -2;
  if (ldqa < heads * (rank + rot)) return -2;
  PrepArgs a{proj, ldp, q_off, dkv_off, norm_w, eps, cos_table, sin_table, positions, row_seq, block_table, table_stride,
             qa, ldqa, qa_is_bf16, heads, dim, rot, rotary, rank, page_size, write_cache};
  hipStream_t s = (hipStream_t)stream;
  if (cache_is_bf16) hipLaunchKernelGGL(latent_prep_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, a, (bf16_t*)cache, (bf16_t*)latent_t);
  else hipLaunchKernelGGL(latent_prep_kernel<float>, dim3(rows), dim3(256), 0, s, a, (float*)cache, (float*)latent_t);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_headwise_linear(const float* x, int ldx, int xhs, const void* wt, int w_is_bf16, int in, int outn,
                                  void* out, int out_is_bf16, int ldo, int ohs, int rows, int heads, void* stream) {
  if (rows <= 0 || heads <= 0 || outn <= 0) return 0;
  if (in <= 0 || (size_t)HL_ROWS * in * sizeof(float) > 48 * 1024) return -2;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((rows + HL_ROWS - 1) / HL_ROWS, heads, (outn + 63) / 64), block(256);
  const size_t bytes = (size_t)HL_ROWS * (in + 4 * 64) * sizeof(float);
  if (w_is_bf16) {
    if (out_is_bf16)
      hipLaunchKernelGGL((headwise_linear_kernel<bf16_t, bf16_t>), grid, block, bytes, s, x, ldx, xhs, (const bf16_t*)wt, in, outn,
                         (bf16_t*)out, ldo, ohs, rows);
    else
      hipLaunchKernelGGL((headwise_linear_kernel<bf16_t, float>), grid, block, bytes, s, x, ldx, xhs, (const bf16_t*)wt, in, outn,
                         (float*)out, ldo, ohs, rows);
  } else {
    if (out_is_bf16)
      hipLaunchKernelGGL((headwise_linear_kernel<float, bf16_t>), grid, block, bytes, s, x, ldx, xhs, (const float*)wt, in, outn,
                         (bf16_t*)out, ldo, ohs, rows);
    else
      hipLaunchKernelGGL((headwise_linear_kernel<float, float>), grid, block, bytes, s, x, ldx, xhs, (const float*)wt, in, outn,
                         (float*)out, ldo, ohs, rows);
  }
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_shared_key_attention(const float* q, int ldq, const int32_t* positions, const int32_t* block_table,
                                       int table_stride, const int32_t* tiles, int num_tiles, const void* cache,
                                       int cache_is_bf16, int num_pages, const float* sink, float* out, int ldo, int heads,
                                       int dk, int dv, int page_size, int window, float scale, int heads_per_group,
                                       void* stream) {
  if (num_tiles <= 0) return 0;
  if (heads <= 0 || dk <= 0 || dv <= 0 || dv > dk || page_size <= 0 || num_pages <= 0) return -2;
  if (heads_per_group != 4 && heads_per_group != 16) return -2;
  if (ldq < heads * dk || ldo < heads * dv) return -2;
  SharedKeyArgs a{q, ldq, positions, block_table, table_stride, tiles, sink, out, ldo, heads, dk, dv, page_size, window,
                  heads_per_group, num_pages, scale};
  hipStream_t s = (hipStream_t)stream;
  if (cache_is_bf16) return launch_shared_key<bf16_t>(a, (const bf16_t*)cache, num_tiles, s);
  return launch_shared_key<float>(a, (const float*)cache, num_tiles, s);
}

// The matrix-core route: bfloat16 cache with key vectors of a multiple of 8 elements, pages of a multiple of 4 slots, and the
// transposed latents beside it.  nsplit > 1 (single-row tiles, 16 heads a group): every wave takes kchunk keys (a multiple
// of 64) and ``partial`` holds tiles * heads * nsplit * (dv + 2) floats.
extern "C" int bw_shared_key_attention_mfma(const void* q, int ldq, const int32_t* positions, const int32_t* block_table,
                                            int table_stride, const int32_t* tiles, int num_tiles, const void* cache,
                                            const void* latent_t, int num_pages, const float* sink, float* out, int ldo,
                                            int heads, int dk, int dv, int page_size, int window, float scale,
                                            int heads_per_group, int nsplit, int kchunk, float* partial,
                                            long long partial_floats, void* stream) {
  if (num_tiles <= 0) return 0;
  if (heads <= 0 || dk <= 0 || (dk % 8) || dv <= 0 || dv > dk || dv > 512 || page_size < 4 || (page_size % 4) || num_pages <= 0) return -2;
  if (heads_per_group < 1 || heads_per_group > 16 || (16 % heads_per_group)) return -2;
  if (ldq < heads * dk || (ldq % 8) || ldo < heads * dv || nsplit < 1 || nsplit > 64) return -2;
  if (reinterpret_cast<uintptr_t>(q) & 15) return -3;
  if (nsplit > 1) {
    if (heads_per_group != 16 || kchunk < 64 || (kchunk % 64) || partial == nullptr) return -2;
    if (partial_floats < (long long)num_tiles * heads * nsplit * (dv + 2)) return -6;
  }
  if ((reinterpret_cast<uintptr_t>(cache) & 15) || (reinterpret_cast<uintptr_t>(latent_t) & 7)) return -3;
  MfmaAttnArgs a{(const bf16_t*)q, ldq, positions, block_table, table_stride, tiles, sink, out, ldo, partial, heads, dk, dv, page_size, window,
                 heads_per_group, num_pages, nsplit, kchunk, scale};
  return launch_shared_key_mfma(a, (const bf16_t*)cache, (const bf16_t*)latent_t, num_tiles, (hipStream_t)stream);
}
