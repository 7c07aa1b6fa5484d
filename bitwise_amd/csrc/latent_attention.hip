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
  float* qa;             // [rows, ldqa]: head h at h * (rank + rot); the rotated part goes to its last rot elements
  int ldqa;
  int heads, dim, rot, rotary, rank, page_size, write_cache;
};

// A workgroup a row.  The rotated part: elements i and i + rotary/2 (i < rotary/2) are a pair; elements from
// ``rotary`` on pass unchanged.
template <typename CT>
__global__ __launch_bounds__(256) void latent_prep_kernel(PrepArgs a, CT* __restrict__ cache) {
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
    a.qa[(size_t)row * a.ldqa + h * width + a.rank + i] = v;
  }
}

// ------------------------------------------------------------------------- a product per head

// out[r][h*ohs + o] = sum_i wt[h][i][o] * x[r][h*xhs + i]: the weights lie input-major, so that neighbouring threads
// (outputs) read neighbouring weights; HL_ROWS rows share every weight that is loaded.  One fused multiply-add chain
// per output, i ascending.
#define HL_ROWS 8
template <typename WT, typename OT>
__global__ __launch_bounds__(256) void headwise_linear_kernel(const float* __restrict__ x, int ldx, int xhs,
                                                              const WT* __restrict__ wt, int in, int outn,
                                                              OT* __restrict__ out, int ldo, int ohs, int rows) {
  extern __shared__ float hl_x[];      // [HL_ROWS][in]
  const int r0 = blockIdx.x * HL_ROWS, h = blockIdx.y;
  const int o = blockIdx.z * 256 + threadIdx.x;
  for (int e = threadIdx.x; e < HL_ROWS * in; e += 256) {
    const int r = e / in, i = e % in;
    hl_x[e] = (r0 + r < rows) ? x[(size_t)(r0 + r) * ldx + h * xhs + i] : 0.0f;
  }
  __syncthreads();
  if (o >= outn) return;
  float acc[HL_ROWS];
#pragma unroll
  for (int r = 0; r < HL_ROWS; ++r) acc[r] = 0.0f;
  const WT* wp = wt + (size_t)h * in * outn + o;
  for (int i = 0; i < in; ++i) {
    const float w = load_f(wp + (size_t)i * outn);
#pragma unroll
    for (int r = 0; r < HL_ROWS; ++r) acc[r] = fmaf(hl_x[r * in + i], w, acc[r]);
  }
#pragma unroll
  for (int r = 0; r < HL_ROWS; ++r)
    if (r0 + r < rows) store_f(out + (size_t)(r0 + r) * ldo + h * ohs + o, acc[r]);
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

}  // namespace

extern "C" int bw_latent_prep(const float* proj, int ldp, int q_off, int dkv_off, const float* norm_w, float eps,
                              const float* cos_table, const float* sin_table, const int32_t* positions,
                              const int32_t* row_seq, const int32_t* block_table, int table_stride, void* cache,
                              int cache_is_bf16, float* qa, int ldqa, int rows, int heads, int dim, int rot, int rotary,
                              int rank, int page_size, int write_cache, void* stream) {
  if (rows <= 0) return 0;
  if (heads <= 0 || dim < 0 || rot < 0 || rotary < 0 || rotary > rot || (rotary & 1) || rank <= 0 || page_size <= 0) return -2;
  if (ldqa < heads * (rank + rot)) return -2;
  PrepArgs a{proj, ldp, q_off, dkv_off, norm_w, eps, cos_table, sin_table, positions, row_seq, block_table, table_stride,
             qa, ldqa, heads, dim, rot, rotary, rank, page_size, write_cache};
  hipStream_t s = (hipStream_t)stream;
  if (cache_is_bf16) hipLaunchKernelGGL(latent_prep_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, a, (bf16_t*)cache);
  else hipLaunchKernelGGL(latent_prep_kernel<float>, dim3(rows), dim3(256), 0, s, a, (float*)cache);
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_headwise_linear(const float* x, int ldx, int xhs, const void* wt, int w_is_bf16, int in, int outn,
                                  void* out, int out_is_bf16, int ldo, int ohs, int rows, int heads, void* stream) {
  if (rows <= 0 || heads <= 0 || outn <= 0) return 0;
  if (in <= 0 || (size_t)HL_ROWS * in * sizeof(float) > 60 * 1024) return -2;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((rows + HL_ROWS - 1) / HL_ROWS, heads, (outn + 255) / 256), block(256);
  const size_t bytes = (size_t)HL_ROWS * in * sizeof(float);
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
