// The row movers fused with their neighbours in the decoder layer (act.py:256-265):
//   rmsnorm_permute_tiled   post-attention RMSNorm + permute into the K-tiled activation matrix of the FFN
//   unpermute_add           unpermute + residual add
//   unpermute_add_rmsnorm   the same, and the RMSNorm that reads the sum next (the following layer's
//                           input_layernorm, act.py:240, or the final norm, act.py:506) as a second output
//   rmsnorm_permute_rows    the same norm with a row-major, expert-sorted result (what the weight gradients of a
//                           training step contract over), and
//   unpermute_rmsnorm_bwd   unpermute of the gradient w.r.t. the normed rows + the norm's backward (+ the residual
//                           branch's gradient), with per-wavefront partial sums of the norm weight's gradient
// Each replaces two (three) passes over [T, H] by one.  bf16 only (the FFN kernels' type).
//
// RMSNorm follows the reference module op by op: x in fp32, variance = mean(x^2), x * rsqrt(variance + eps),
// rounded to bf16, times the bf16 weight, rounded to bf16 (Qwen2RMSNorm as used at act.py:190-193).  The sum of
// squares is accumulated in fp32 in this kernel's own order, so results can differ from eager PyTorch in the last
// bf16 bit where a value sits on a rounding boundary.
#include "common.h"
#include "tiled_layout.h"

namespace wx {
namespace {

constexpr int kSplit = 4;        // wavefronts per 16-row block = one workgroup; each takes a quarter of the columns
constexpr int kMaxChunks = 32;   // column blocks per wavefront held in registers (hidden <= 4096)

__device__ __forceinline__ u32x4 ld16(const u32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st16(u32x4* p, const u32x4& v) { __builtin_nontemporal_store(v, p); }

// NCH = column blocks per wavefront (compile-time so the row stays in registers)
template <int NCH>
__global__ __launch_bounds__(kSplit * 64) void rmsnorm_permute_tiled_kernel(
    const u32x4* __restrict__ x, const u32x4* __restrict__ weight, float eps, unsigned char* __restrict__ out,
    const int32_t* __restrict__ sorted_row_id, const int32_t* __restrict__ expert_offsets, int64_t num_tokens,
    int64_t row_blocks) {
  __shared__ float s_part[kSplit][kBlkRows];
  const int lane = threadIdx.x & 63, part = threadIdx.x >> 6;
  const int64_t rb = blockIdx.x;
  const int32_t o0 = expert_offsets[0], o1 = expert_offsets[1], o2 = expert_offsets[2];
  const int64_t pad0 = round_up_256(o1 - o0);
  // lane -> (row of the block, 16-byte slot); the slot holds chunk slot ^ ((row >> 2) & 3) of the 32 columns
  const int r = lane >> 2, slot = lane & 3, chunk = slot ^ ((r >> 2) & 3);
  const int64_t prow = rb * kBlkRows + r;
  int64_t pos = -1;  // padded row -> sorted position (none for the padding rows of either expert)
  if (prow < pad0) { if (prow < o1 - o0) pos = o0 + prow; }
  else if (prow - pad0 < o2 - o1) pos = o1 + (prow - pad0);
  const int64_t src_tok = (pos >= 0 && pos < num_tokens) ? sorted_row_id[pos] : -1;
  constexpr int64_t kChunksPerRow = static_cast<int64_t>(NCH) * kSplit * 4;
  const int kb0 = part * NCH;  // first column block of this wavefront
  const u32x4* src = x + (src_tok < 0 ? 0 : src_tok) * kChunksPerRow + kb0 * 4 + chunk;
  u32x4 v[NCH];
#pragma unroll
  for (int u = 0; u < NCH; ++u) v[u] = src_tok < 0 ? u32x4{0, 0, 0, 0} : ld16(src + u * 4);
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    float f[8];
    unpack16<WX_BF16>(v[u], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
  }
  // the 4 lanes of a row, then the 4 wavefronts of the workgroup
  ss += __shfl_xor(ss, 1);
  ss += __shfl_xor(ss, 2);
  if (slot == 0) s_part[part][r] = ss;
  __syncthreads();
  const float total = s_part[0][r] + s_part[1][r] + s_part[2][r] + s_part[3][r];
  const float inv = __frsqrt_rn(total / static_cast<float>(kChunksPerRow * 8) + eps);
  unsigned char* dst = out + (rb << 10) + lane * 16;
#pragma unroll
  for (int u = 0; u < NCH; ++u) {
    float f[8], w[8];
    unpack16<WX_BF16>(v[u], f);
    unpack16<WX_BF16>(weight[(kb0 + u) * 4 + chunk], w);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = w[e] * round_bf16(f[e] * inv);  // pack16 rounds the product
    st16(reinterpret_cast<u32x4*>(dst + ((static_cast<int64_t>(kb0 + u) * row_blocks) << 10)), pack16<WX_BF16>(f));
  }
}

// The same with 128-byte reads: a lane takes chunk (lane & 7) of the 128 bytes spanning a PAIR of column blocks, for
// rows (lane >> 3) and (lane >> 3) + 8 of the row block (a load instruction touches 8 rows x a whole cache line
// instead of 16 rows x half a line; a store instruction writes two 512-byte runs).  NP = pairs of column blocks per
// wavefront.
template <int NP>
__global__ __launch_bounds__(kSplit * 64) void rmsnorm_permute_tiled128_kernel(
    const u32x4* __restrict__ x, const u32x4* __restrict__ weight, float eps, unsigned char* __restrict__ out,
    const int32_t* __restrict__ sorted_row_id, const int32_t* __restrict__ expert_offsets, int64_t num_tokens,
    int64_t row_blocks) {
  __shared__ float s_part[kSplit][kBlkRows];
  const int lane = threadIdx.x & 63, part = threadIdx.x >> 6;
  const int64_t rb = blockIdx.x;
  const int32_t o0 = expert_offsets[0], o1 = expert_offsets[1], o2 = expert_offsets[2];
  const int64_t pad0 = round_up_256(o1 - o0);
  const int r8 = lane >> 3, c8 = lane & 7;
  constexpr int64_t kChunksPerRow = static_cast<int64_t>(NP) * 2 * kSplit * 4;
  const int pair0 = part * NP;  // first pair of column blocks of this wavefront
  u32x4 v[NP][2];
  bool live[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t prow = rb * kBlkRows + 8 * h + r8;
    int64_t pos = -1;
    if (prow < pad0) { if (prow < o1 - o0) pos = o0 + prow; }
    else if (prow - pad0 < o2 - o1) pos = o1 + (prow - pad0);
    const int64_t tok = (pos >= 0 && pos < num_tokens) ? sorted_row_id[pos] : -1;
    live[h] = tok >= 0;
    const u32x4* src = x + (tok < 0 ? 0 : tok) * kChunksPerRow + pair0 * 8 + c8;
#pragma unroll
    for (int u = 0; u < NP; ++u) v[u][h] = live[h] ? ld16(src + u * 8) : u32x4{0, 0, 0, 0};
  }
  float inv[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NP; ++u) {
      float f[8];
      unpack16<WX_BF16>(v[u][h], f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
    }
    ss += __shfl_xor(ss, 1);
    ss += __shfl_xor(ss, 2);
    ss += __shfl_xor(ss, 4);  // the 8 lanes of a row
    if (c8 == 0) s_part[part][8 * h + r8] = ss;
  }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = 8 * h + r8;
    const float total = s_part[0][r] + s_part[1][r] + s_part[2][r] + s_part[3][r];
    inv[h] = __frsqrt_rn(total / static_cast<float>(kChunksPerRow * 8) + eps);
  }
  unsigned char* base = out + (rb << 10) + (((c8 >> 2) * row_blocks) << 10);  // first or second block of the pair
#pragma unroll
  for (int u = 0; u < NP; ++u) {
    float w[8];
    unpack16<WX_BF16>(weight[(pair0 + u) * 8 + c8], w);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = 8 * h + r8;
      float f[8];
      unpack16<WX_BF16>(v[u][h], f);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = w[e] * round_bf16(f[e] * inv[h]);  // pack16 rounds the product
      const int off = r * 64 + (((c8 & 3) ^ ((r >> 2) & 3)) << 4);
      st16(reinterpret_cast<u32x4*>(base + ((static_cast<int64_t>(pair0 + u) * 2 * row_blocks) << 10) + off), pack16<WX_BF16>(f));
    }
  }
}

// out[t] = resid[t] + y[row_id_map[t]] (resid[t] alone when the map entry is -1); one wavefront per destination row.
__global__ __launch_bounds__(256) void unpermute_add_kernel(const u32x4* __restrict__ y, const u32x4* __restrict__ resid,
                                                            u32x4* __restrict__ out, const int32_t* __restrict__ row_id_map,
                                                            int64_t num_tokens, int64_t vec_per_row) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * 4;
  for (int64_t t = wave; t < num_tokens; t += n_waves) {
    const int32_t src_row = row_id_map[t];
    const u32x4* src = y + static_cast<int64_t>(src_row < 0 ? 0 : src_row) * vec_per_row;
    const u32x4* res = resid + t * vec_per_row;
    u32x4* dst = out + t * vec_per_row;
    for (int64_t c = lane; c < vec_per_row; c += 4 * 64) {
      u32x4 a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t cc = c + u * 64;
        if (cc < vec_per_row) {
          a[u] = ld16(res + cc);
          b[u] = src_row < 0 ? u32x4{0, 0, 0, 0} : ld16(src + cc);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t cc = c + u * 64;
        if (cc < vec_per_row) {
          float fa[8], fb[8];
          unpack16<WX_BF16>(a[u], fa);
          unpack16<WX_BF16>(b[u], fb);
#pragma unroll
          for (int e = 0; e < 8; ++e) fa[e] += fb[e];
          st16(dst + cc, pack16<WX_BF16>(fa));
        }
      }
    }
  }
}

// out[t] = resid[t] + y[row_id_map[t]], normed[t] = weight * rmsnorm(out[t]); one wavefront per row, the row held
// in registers (NV 16-byte chunks per lane).  The norm reads the bf16-rounded sum, as a separate kernel would.
template <int NV>
__global__ __launch_bounds__(256) void unpermute_add_rmsnorm_kernel(
    const u32x4* __restrict__ y, const u32x4* __restrict__ resid, u32x4* __restrict__ out, u32x4* __restrict__ normed,
    const u32x4* __restrict__ weight, float eps, const int32_t* __restrict__ row_id_map, int64_t num_tokens,
    int vec_per_row) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * 4;
  for (int64_t t = wave; t < num_tokens; t += n_waves) {
    const int32_t src_row = row_id_map[t];
    const u32x4* src = y + static_cast<int64_t>(src_row < 0 ? 0 : src_row) * vec_per_row;
    const u32x4* res = resid + t * vec_per_row;
    u32x4 a[NV], b[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int cc = lane + u * 64;
      if (cc < vec_per_row) {
        a[u] = ld16(res + cc);
        b[u] = src_row < 0 ? u32x4{0, 0, 0, 0} : ld16(src + cc);
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      if (lane + u * 64 < vec_per_row) {
        float fa[8], fb[8];
        unpack16<WX_BF16>(a[u], fa);
        unpack16<WX_BF16>(b[u], fb);
#pragma unroll
        for (int e = 0; e < 8; ++e) fa[e] += fb[e];
        a[u] = pack16<WX_BF16>(fa);  // the residual stream as stored
        st16(out + t * vec_per_row + lane + u * 64, a[u]);
        unpack16<WX_BF16>(a[u], fa);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += fa[e] * fa[e];
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
    const float inv = __frsqrt_rn(ss / static_cast<float>(vec_per_row * 8) + eps);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int cc = lane + u * 64;
      if (cc < vec_per_row) {
        float f[8], w[8];
        unpack16<WX_BF16>(a[u], f);
        unpack16<WX_BF16>(weight[cc], w);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = w[e] * round_bf16(f[e] * inv);  // pack16 rounds the product
        st16(normed + t * vec_per_row + cc, pack16<WX_BF16>(f));
      }
    }
  }
}

// out[pos] = weight * rmsnorm(x[sorted_row_id[pos]]), row-major in expert-sorted order; one wavefront per row, the
// row held in registers.  The same arithmetic as the tiled form above.
template <int NV>
__global__ __launch_bounds__(256) void rmsnorm_permute_rows_kernel(
    const u32x4* __restrict__ x, const u32x4* __restrict__ weight, float eps, u32x4* __restrict__ out,
    const int32_t* __restrict__ sorted_row_id, int64_t num_tokens, int vec_per_row) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * 4;
  for (int64_t pos = wave; pos < num_tokens; pos += n_waves) {
    const int32_t tok = sorted_row_id[pos];
    const bool live = tok >= 0 && tok < num_tokens;
    const u32x4* src = x + static_cast<int64_t>(live ? tok : 0) * vec_per_row;
    u32x4 a[NV];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int cc = lane + u * 64;
      a[u] = (cc < vec_per_row && live) ? ld16(src + cc) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      float f[8];
      unpack16<WX_BF16>(a[u], f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
    const float inv = __frsqrt_rn(ss / static_cast<float>(vec_per_row * 8) + eps);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int cc = lane + u * 64;
      if (cc < vec_per_row) {
        float f[8], w[8];
        unpack16<WX_BF16>(a[u], f);
        unpack16<WX_BF16>(weight[cc], w);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = w[e] * round_bf16(f[e] * inv);  // pack16 rounds the product
        st16(out + pos * vec_per_row + cc, pack16<WX_BF16>(f));
      }
    }
  }
}

// Backward of  y[row_id_map[t]] = weight * rmsnorm(x[t])  for the gradient g of the sorted rows:
//   dx[t] = (add[t] +) inv * (g w - xhat * mean(g w xhat)),  xhat = x[t] * inv,  inv = rsqrt(mean(x[t]^2) + eps)
// in fp32 with one rounding at the store (a dropped token, map entry -1, has g = 0), and
//   dw_partial[wavefront] = sum over the wavefront's rows of g * round_bf16(xhat)   (the forward's rounded xhat),
// fp32 [number of wavefronts, H]; a second kernel adds the partials up.  One wavefront per token row.
template <int NV>
__global__ __launch_bounds__(256) void unpermute_rmsnorm_bwd_kernel(
    const u32x4* __restrict__ g_sorted, const u32x4* __restrict__ x, const u32x4* __restrict__ weight, float eps,
    const u32x4* __restrict__ add, u32x4* __restrict__ dx, float* __restrict__ dw_partial,
    const int32_t* __restrict__ row_id_map, int64_t num_tokens, int vec_per_row) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * 4;
  float dw[NV][8];
#pragma unroll
  for (int u = 0; u < NV; ++u)
#pragma unroll
    for (int e = 0; e < 8; ++e) dw[u][e] = 0.f;
  for (int64_t t = wave; t < num_tokens; t += n_waves) {
    const int32_t src_row = row_id_map[t];
    const u32x4* gsrc = g_sorted + static_cast<int64_t>(src_row < 0 ? 0 : src_row) * vec_per_row;
    u32x4 xv[NV], gv[NV], av[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int cc = lane + u * 64;
      const bool in = cc < vec_per_row;
      xv[u] = in ? ld16(x + t * vec_per_row + cc) : u32x4{0, 0, 0, 0};
      gv[u] = (in && src_row >= 0) ? ld16(gsrc + cc) : u32x4{0, 0, 0, 0};
      av[u] = (in && add != nullptr) ? ld16(add + t * vec_per_row + cc) : u32x4{0, 0, 0, 0};
    }
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      float f[8];
      unpack16<WX_BF16>(xv[u], f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
    const float inv = __frsqrt_rn(ss / static_cast<float>(vec_per_row * 8) + eps);
    float dot = 0.f;  // sum of g w xhat over the row
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int cc = lane + u * 64;
      if (cc < vec_per_row) {
        float xf[8], gf[8], w[8];
        unpack16<WX_BF16>(xv[u], xf);
        unpack16<WX_BF16>(gv[u], gf);
        unpack16<WX_BF16>(weight[cc], w);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xhat = xf[e] * inv;
          dw[u][e] += gf[e] * round_bf16(xhat);
          dot += gf[e] * w[e] * xhat;
        }
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
    const float mean = dot / static_cast<float>(vec_per_row * 8);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int cc = lane + u * 64;
      if (cc < vec_per_row) {
        float xf[8], gf[8], af[8], w[8];
        unpack16<WX_BF16>(xv[u], xf);
        unpack16<WX_BF16>(gv[u], gf);
        unpack16<WX_BF16>(av[u], af);
        unpack16<WX_BF16>(weight[cc], w);
#pragma unroll
        for (int e = 0; e < 8; ++e) af[e] += inv * (gf[e] * w[e] - xf[e] * inv * mean);
        st16(dx + t * vec_per_row + cc, pack16<WX_BF16>(af));
      }
    }
  }
  float* mine = dw_partial + wave * (static_cast<int64_t>(vec_per_row) * 8);
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int cc = lane + u * 64;
    if (cc < vec_per_row) {
#pragma unroll
      for (int e = 0; e < 8; ++e) mine[cc * 8 + e] = dw[u][e];
    }
  }
}

// dw[c] = sum over p of partial[p][c], rounded to bf16.  A workgroup takes 64 columns; its four wavefronts split the
// partial rows and meet in LDS.
__global__ __launch_bounds__(256) void column_sums_kernel(const float* __restrict__ partial, __bf16* __restrict__ dw,
                                                          int64_t n_partials, int64_t cols) {
  __shared__ float s_sum[4][64];
  const int lane = threadIdx.x & 63, part = threadIdx.x >> 6;
  const int64_t c = static_cast<int64_t>(blockIdx.x) * 64 + lane;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < cols) {
    int64_t p = part;
    for (; p + 12 < n_partials; p += 16) {
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] += partial[(p + 4 * u) * cols + c];
    }
    for (; p < n_partials; p += 4) acc[0] += partial[p * cols + c];
  }
  s_sum[part][lane] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  __syncthreads();
  if (part == 0 && c < cols) dw[c] = static_cast<__bf16>((s_sum[0][lane] + s_sum[1][lane]) + (s_sum[2][lane] + s_sum[3][lane]));
}

}  // namespace
}  // namespace wx

using namespace wx;

extern "C" int wx_rmsnorm_permute_rows_tiled(const void* x, const void* weight, float eps, void* out_tiled,
                                             const int32_t* sorted_row_id, const int32_t* expert_offsets,
                                             int64_t num_tokens, int64_t num_cols, wx_stream_t stream) {
  const char* who = "wx_rmsnorm_permute_rows_tiled";
  if (num_tokens < 0 || num_cols <= 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad sizes", who);
  if (num_cols % (kBlkCols * kSplit) != 0 || num_cols / (kBlkCols * kSplit) > kMaxChunks)
    return fail(WX_ERR_UNSUPPORTED, "%s: num_cols (%lld) must be a multiple of %d and at most %d", who,
                static_cast<long long>(num_cols), kBlkCols * kSplit, kBlkCols * kSplit * kMaxChunks);
  if (!(eps >= 0.f)) return fail(WX_ERR_INVALID_ARGUMENT, "%s: eps must be non-negative", who);
  if (num_tokens == 0) return WX_OK;
  if (num_tokens > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", who);
  if (!x || !weight || !out_tiled || !sorted_row_id || !expert_offsets)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out_tiled)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  const int64_t row_blocks = padded_sorted_rows(num_tokens) / kBlkRows;
  const int nch = static_cast<int>(num_cols / (kBlkCols * kSplit));
  const dim3 grid(static_cast<unsigned>(row_blocks)), block(kSplit * 64);
  hipStream_t s = as_stream(stream);
#define WX_CASE(N)                                                                                                  \
  case N:                                                                                                           \
    hipLaunchKernelGGL(rmsnorm_permute_tiled_kernel<N>, grid, block, 0, s, static_cast<const u32x4*>(x),            \
                       static_cast<const u32x4*>(weight), eps, static_cast<unsigned char*>(out_tiled), sorted_row_id, \
                       expert_offsets, num_tokens, row_blocks);                                                     \
    break;
#define WX_CASE128(N)                                                                                               \
  case 2 * N:                                                                                                       \
    hipLaunchKernelGGL(rmsnorm_permute_tiled128_kernel<N>, grid, block, 0, s, static_cast<const u32x4*>(x),         \
                       static_cast<const u32x4*>(weight), eps, static_cast<unsigned char*>(out_tiled), sorted_row_id, \
                       expert_offsets, num_tokens, row_blocks);                                                     \
    return check_launch("rmsnorm_permute_tiled128_kernel");
  switch (nch) {  // an even number of column blocks per wavefront: the form with whole-line reads
    WX_CASE128(1) WX_CASE128(2) WX_CASE128(3) WX_CASE128(4) WX_CASE128(5) WX_CASE128(6) WX_CASE128(7) WX_CASE128(8)
    WX_CASE128(10) WX_CASE128(12) WX_CASE128(14) WX_CASE128(16)
    default: break;
  }
#undef WX_CASE128
  switch (nch) {
    WX_CASE(1) WX_CASE(2) WX_CASE(3) WX_CASE(4) WX_CASE(5) WX_CASE(6) WX_CASE(7) WX_CASE(8)
    WX_CASE(9) WX_CASE(10) WX_CASE(11) WX_CASE(12) WX_CASE(13) WX_CASE(14) WX_CASE(15) WX_CASE(16)
    WX_CASE(20) WX_CASE(24) WX_CASE(28) WX_CASE(32)
    default:
      return fail(WX_ERR_UNSUPPORTED, "%s: num_cols %lld has no built kernel (hidden / 128 must be 1..16, 20, 24, 28 or 32)",
                  who, static_cast<long long>(num_cols));
  }
#undef WX_CASE
  return check_launch("rmsnorm_permute_tiled_kernel");
}

extern "C" int wx_unpermute_rows_add(const void* y, const void* residual, void* out, const int32_t* row_id_map,
                                     int64_t num_tokens, int64_t num_cols, wx_stream_t stream) {
  const char* who = "wx_unpermute_rows_add";
  if (num_tokens < 0 || num_cols <= 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad sizes", who);
  if (num_cols % 8 != 0) return fail(WX_ERR_UNSUPPORTED, "%s: num_cols must be a multiple of 8", who);
  if (num_tokens == 0) return WX_OK;
  if (num_tokens > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", who);
  if (!y || !residual || !out || !row_id_map) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(out)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  const int64_t want = (num_tokens + 3) / 4;
  const int64_t cap = static_cast<int64_t>(device_cu_count()) * 8;  // 8 workgroups of 4 wavefronts per CU cover HBM latency
  hipLaunchKernelGGL(unpermute_add_kernel, dim3(static_cast<unsigned>(want < cap ? want : cap)), dim3(256), 0,
                     as_stream(stream), static_cast<const u32x4*>(y), static_cast<const u32x4*>(residual),
                     static_cast<u32x4*>(out), row_id_map, num_tokens, num_cols / 8);
  return check_launch("unpermute_add_kernel");
}

extern "C" int wx_unpermute_rows_add_rmsnorm(const void* y, const void* residual, void* out, void* normed,
                                             const void* weight, float eps, const int32_t* row_id_map,
                                             int64_t num_tokens, int64_t num_cols, wx_stream_t stream) {
  const char* who = "wx_unpermute_rows_add_rmsnorm";
  if (num_tokens < 0 || num_cols <= 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad sizes", who);
  if (num_cols % 8 != 0 || num_cols > 4096)
    return fail(WX_ERR_UNSUPPORTED, "%s: num_cols (%lld) must be a multiple of 8 and at most 4096", who,
                static_cast<long long>(num_cols));
  if (!(eps >= 0.f)) return fail(WX_ERR_INVALID_ARGUMENT, "%s: eps must be non-negative", who);
  if (num_tokens == 0) return WX_OK;
  if (num_tokens > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", who);
  if (!y || !residual || !out || !normed || !weight || !row_id_map)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(out) |
       reinterpret_cast<uintptr_t>(normed) | reinterpret_cast<uintptr_t>(weight)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  const int vec = static_cast<int>(num_cols / 8);
  const int64_t want = (num_tokens + 3) / 4;
  const int64_t cap = static_cast<int64_t>(device_cu_count()) * 8;
  const dim3 grid(static_cast<unsigned>(want < cap ? want : cap)), block(256);
  hipStream_t s = as_stream(stream);
#define WX_CASE(N)                                                                                                   \
  case N:                                                                                                            \
    hipLaunchKernelGGL(unpermute_add_rmsnorm_kernel<N>, grid, block, 0, s, static_cast<const u32x4*>(y),             \
                       static_cast<const u32x4*>(residual), static_cast<u32x4*>(out), static_cast<u32x4*>(normed),   \
                       static_cast<const u32x4*>(weight), eps, row_id_map, num_tokens, vec);                         \
    break;
  switch ((vec + 63) / 64) {
    WX_CASE(1) WX_CASE(2) WX_CASE(3) WX_CASE(4) WX_CASE(5) WX_CASE(6) WX_CASE(7) WX_CASE(8)
    default: return fail(WX_ERR_UNSUPPORTED, "%s: num_cols too large", who);
  }
#undef WX_CASE
  return check_launch("unpermute_add_rmsnorm_kernel");
}

extern "C" int wx_rmsnorm_permute_rows(const void* x, const void* weight, float eps, void* out_sorted,
                                       const int32_t* sorted_row_id, int64_t num_tokens, int64_t num_cols,
                                       wx_stream_t stream) {
  const char* who = "wx_rmsnorm_permute_rows";
  if (num_tokens < 0 || num_cols <= 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad sizes", who);
  if (num_cols % 8 != 0 || num_cols > 4096)
    return fail(WX_ERR_UNSUPPORTED, "%s: num_cols (%lld) must be a multiple of 8 and at most 4096", who,
                static_cast<long long>(num_cols));
  if (!(eps >= 0.f)) return fail(WX_ERR_INVALID_ARGUMENT, "%s: eps must be non-negative", who);
  if (num_tokens == 0) return WX_OK;
  if (num_tokens > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", who);
  if (!x || !weight || !out_sorted || !sorted_row_id) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out_sorted)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  const int vec = static_cast<int>(num_cols / 8);
  const int64_t want = (num_tokens + 3) / 4;
  const int64_t cap = static_cast<int64_t>(device_cu_count()) * 8;
  const dim3 grid(static_cast<unsigned>(want < cap ? want : cap)), block(256);
  hipStream_t s = as_stream(stream);
#define WX_CASE(N)                                                                                                   \
  case N:                                                                                                            \
    hipLaunchKernelGGL(rmsnorm_permute_rows_kernel<N>, grid, block, 0, s, static_cast<const u32x4*>(x),              \
                       static_cast<const u32x4*>(weight), eps, static_cast<u32x4*>(out_sorted), sorted_row_id,       \
                       num_tokens, vec);                                                                             \
    break;
  switch ((vec + 63) / 64) {
    WX_CASE(1) WX_CASE(2) WX_CASE(3) WX_CASE(4) WX_CASE(5) WX_CASE(6) WX_CASE(7) WX_CASE(8)
    default: return fail(WX_ERR_UNSUPPORTED, "%s: num_cols too large", who);
  }
#undef WX_CASE
  return check_launch("rmsnorm_permute_rows_kernel");
}

extern "C" size_t wx_rmsnorm_bwd_workspace_bytes(int64_t num_cols) {
  if (num_cols <= 0) return 0;
  // one fp32 row of partial weight-gradient sums per wavefront of the largest grid the backward launches
  return static_cast<size_t>(device_cu_count()) * 2 * 4 * static_cast<size_t>(num_cols) * sizeof(float);
}

extern "C" int wx_unpermute_rows_rmsnorm_bwd(const void* grad_sorted, const void* x, const void* weight, float eps,
                                             const void* add, void* grad_x, void* grad_weight,
                                             const int32_t* row_id_map, int64_t num_tokens, int64_t num_cols,
                                             void* workspace, size_t workspace_bytes, wx_stream_t stream) {
  const char* who = "wx_unpermute_rows_rmsnorm_bwd";
  if (num_tokens < 0 || num_cols <= 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad sizes", who);
  if (num_cols % 8 != 0 || num_cols > 4096)
    return fail(WX_ERR_UNSUPPORTED, "%s: num_cols (%lld) must be a multiple of 8 and at most 4096", who,
                static_cast<long long>(num_cols));
  if (!(eps >= 0.f)) return fail(WX_ERR_INVALID_ARGUMENT, "%s: eps must be non-negative", who);
  if (num_tokens > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", who);
  if (!grad_weight || !workspace) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if (num_tokens > 0 && (!grad_sorted || !x || !weight || !grad_x || !row_id_map))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((reinterpret_cast<uintptr_t>(grad_sorted) | reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) |
       reinterpret_cast<uintptr_t>(add) | reinterpret_cast<uintptr_t>(grad_x) | reinterpret_cast<uintptr_t>(workspace)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  if (workspace_bytes < wx_rmsnorm_bwd_workspace_bytes(num_cols))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: workspace too small (see wx_rmsnorm_bwd_workspace_bytes)", who);
  const int vec = static_cast<int>(num_cols / 8);
  const int64_t want = (num_tokens + 3) / 4;
  const int64_t cap = static_cast<int64_t>(device_cu_count()) * 2;  // bounded by the workspace: one partial row per wavefront
  const int64_t blocks = want < cap ? (want > 0 ? want : 1) : cap;
  const dim3 grid(static_cast<unsigned>(blocks)), block(256);
  hipStream_t s = as_stream(stream);
#define WX_CASE(N)                                                                                                   \
  case N:                                                                                                            \
    hipLaunchKernelGGL(unpermute_rmsnorm_bwd_kernel<N>, grid, block, 0, s, static_cast<const u32x4*>(grad_sorted),   \
                       static_cast<const u32x4*>(x), static_cast<const u32x4*>(weight), eps,                        \
                       static_cast<const u32x4*>(add), static_cast<u32x4*>(grad_x), static_cast<float*>(workspace), \
                       row_id_map, num_tokens, vec);                                                                 \
    break;
  switch ((vec + 63) / 64) {
    WX_CASE(1) WX_CASE(2) WX_CASE(3) WX_CASE(4) WX_CASE(5) WX_CASE(6) WX_CASE(7) WX_CASE(8)
    default: return fail(WX_ERR_UNSUPPORTED, "%s: num_cols too large", who);
  }
#undef WX_CASE
  if (int rc = check_launch("unpermute_rmsnorm_bwd_kernel")) return rc;
  hipLaunchKernelGGL(column_sums_kernel, dim3(static_cast<unsigned>((num_cols + 63) / 64)), dim3(256), 0, s,
                     static_cast<const float*>(workspace), static_cast<__bf16*>(grad_weight), blocks * 4, num_cols);
  return check_launch("column_sums_kernel");
}

extern "C" int wx_moe_block_forward(const void* x, void* out, const int32_t* row_id_map, const int32_t* sorted_row_id,
                                    const int32_t* expert_offsets, const void* gate0, const void* up0,
                                    const void* down0, const void* gate1, const void* up1, const void* down1,
                                    void* x_tiled, void* hmid, int64_t num_rows, int64_t hidden, int64_t inter0,
                                    int64_t inter1, const int64_t* host_rows_per_expert, const void* norm_weight,
                                    float eps, int add_residual, void* ffn_workspace, wx_stream_t stream) {
  const char* who = "wx_moe_block_forward";
  if (num_rows < 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: negative row count", who);
  if (num_rows == 0) return WX_OK;
  if (!sorted_row_id) return fail(WX_ERR_INVALID_ARGUMENT, "%s: sorted_row_id is required", who);
  if (ffn_workspace != nullptr && norm_weight == nullptr)
    // one launch for the permute and both GEMMs where the shape allows it, else the launches below
    return wx_dual_swiglu_ffn_fused(x, x_tiled, out, add_residual ? x : nullptr, expert_offsets, gate0, up0, down0, gate1,
                                    up1, down1, hmid, num_rows, hidden, inter0, inter1, host_rows_per_expert,
                                    sorted_row_id, ffn_workspace, stream);
  if (int rc = norm_weight != nullptr
                   ? wx_rmsnorm_permute_rows_tiled(x, norm_weight, eps, x_tiled, sorted_row_id, expert_offsets, num_rows,
                                                   hidden, stream)
                   : wx_permute_rows_tiled(x, x_tiled, row_id_map, sorted_row_id, expert_offsets, num_rows, hidden,
                                           stream))
    return rc;
  if (ffn_workspace != nullptr)  // one launch for both GEMMs where the shape allows it, else the two below
    return wx_dual_swiglu_ffn_fused(nullptr, x_tiled, out, add_residual ? x : nullptr, expert_offsets, gate0, up0, down0,
                                    gate1, up1, down1, hmid, num_rows, hidden, inter0, inter1, host_rows_per_expert,
                                    sorted_row_id, ffn_workspace, stream);
  if (int rc = wx_dual_swiglu_gate_up(x_tiled, hmid, expert_offsets, gate0, up0, gate1, up1, num_rows, hidden, inter0,
                                      inter1, host_rows_per_expert, stream))
    return rc;
  if (add_residual)
    return wx_dual_down_proj_residual(hmid, out, x, expert_offsets, down0, down1, num_rows, hidden, inter0, inter1,
                                      host_rows_per_expert, sorted_row_id, stream);
  return wx_dual_down_proj(hmid, out, expert_offsets, down0, down1, num_rows, hidden, inter0, inter1,
                           host_rows_per_expert, sorted_row_id, stream);
}
