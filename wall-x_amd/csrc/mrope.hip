// 3D multimodal RoPE apply (forward and adjoint) for gfx950.
//
// HBM-bound elementwise kernels.
//
// mrope_rows_kernel (the one the model shapes use): a thread owns one 16-byte chunk position of the head
// (channels [8c, 8c+8) for 2-byte types) of one token and walks over ALL heads of q and k.  It loads the selected
// cos/sin values of its channels once, gets the partner chunk of every rotation (the same channels in the other
// half of the head) from the lane that owns it through a lane exchange, and writes its own 16 bytes.  The lanes
// of a token cover a whole head, so a wavefront reads whole 256-byte heads and writes runs of consecutive tokens
// (1 KiB for head_dim 128) of the head-major output; the loads of several heads are in flight before the first
// result is needed.
//
// mrope_kernel (general fallback: head sizes whose chunk count is not a power of two, sections that cut through
// a chunk): a thread owns the 8 channels [8j, 8j+8) of the low half together with their partners in the high
// half and applies them to a few heads.
//
// q/k/outputs are addressed through (batch, head, seq) strides so the projection's [B, S, H, D] memory is read
// in place.
#include "common.h"

namespace wx {
namespace {

constexpr int kMaxHeadDim = 256;

struct AxisTable {
  uint8_t axis[kMaxHeadDim];        // position plane (0 t, 1 h, 2 w) per channel
  uint8_t uniform[kMaxHeadDim / 8]; // 1 when the 8 channels starting at 8*i share one plane
};

struct Strides {
  int64_t b, h, s;
};

template <int DT>
__device__ __forceinline__ void load8(const void* base, int64_t elem_off, float* f) {
  if constexpr (DT == WX_F32) {
    const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const float*>(base) + elem_off);
    unpack16<DT>(__builtin_nontemporal_load(p), f);
    unpack16<DT>(__builtin_nontemporal_load(p + 1), f + 4);
  } else {
    unpack16<DT>(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + elem_off)), f);
  }
}
// same as load8 with a regular (cached) load: the cos/sin chunks are re-read by every head group
template <int DT>
__device__ __forceinline__ void load8_cached(const void* base, int64_t elem_off, float* f) {
  if constexpr (DT == WX_F32) {
    const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const float*>(base) + elem_off);
    unpack16<DT>(p[0], f);
    unpack16<DT>(p[1], f + 4);
  } else {
    unpack16<DT>(*reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(base) + elem_off), f);
  }
}
template <int DT>
__device__ __forceinline__ void store8(void* base, int64_t elem_off, const float* f) {
  if constexpr (DT == WX_F32) {
    u32x4* p = reinterpret_cast<u32x4*>(static_cast<float*>(base) + elem_off);
    __builtin_nontemporal_store(pack16<DT>(f), p);
    __builtin_nontemporal_store(pack16<DT>(f + 4), p + 1);
  } else {
    __builtin_nontemporal_store(pack16<DT>(f), reinterpret_cast<u32x4*>(static_cast<uint16_t*>(base) + elem_off));
  }
}
template <int DT>
__device__ __forceinline__ float load1(const void* base, int64_t elem_off) {
  if constexpr (DT == WX_F32) return static_cast<const float*>(base)[elem_off];
  else return Elem<DT>::load(static_cast<const uint16_t*>(base)[elem_off]);
}

// cos/sin for channels [d0, d0+8) of one token, each channel from its own position plane.
template <int DT>
__device__ __forceinline__ void load_selected(const void* table, const AxisTable& ax, int64_t plane_stride,
                                              int64_t token_off, int d0, float* f) {
  if (ax.uniform[d0 >> 3]) {
    load8_cached<DT>(table, ax.axis[d0] * plane_stride + token_off + d0, f);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = load1<DT>(table, ax.axis[d0 + e] * plane_stride + token_off + d0 + e);
  }
}

// Heads per thread: the loads of all of them are issued before the first result is needed.
#ifndef WX_MROPE_HPT
#define WX_MROPE_HPT 3
#endif
constexpr int kHeadsPerThread = WX_MROPE_HPT;

template <int DT, bool BWD>
__global__ __launch_bounds__(256) void mrope_kernel(
    const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ cos_t,
    const void* __restrict__ sin_t, void* __restrict__ q_out, void* __restrict__ k_out, int64_t n_tokens,
    int64_t seq, int n_q_heads, int n_kv_heads, int head_dim, Strides sq, Strides sk, Strides sqo, Strides sko,
    AxisTable ax) {
  const int groups = head_dim / 16;  // rotation groups per head
  // blockIdx.y = head group (uniform per workgroup), blockIdx.x walks (token, rotation group)
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int j = static_cast<int>(gid % groups);
  const int64_t token = gid / groups;
  if (token >= n_tokens) return;
  const int h0 = blockIdx.y * kHeadsPerThread;
  const int64_t b = token / seq, s = token - b * seq;
  const int half = head_dim / 2;
  const int d_lo = 8 * j, d_hi = half + 8 * j;
  const int64_t plane = n_tokens * head_dim, tok_off = token * head_dim;
  const int n_heads = n_q_heads + n_kv_heads;

  float x_lo[kHeadsPerThread][8], x_hi[kHeadsPerThread][8];
#pragma unroll
  for (int u = 0; u < kHeadsPerThread; ++u) {
    const int h = h0 + u;
    if (h < n_heads) {
      const bool is_q = h < n_q_heads;
      const int hh = is_q ? h : h - n_q_heads;
      const Strides& si = is_q ? sq : sk;
      const void* in = is_q ? q : k;
      const int64_t in_off = b * si.b + hh * si.h + s * si.s;
      load8<DT>(in, in_off + d_lo, x_lo[u]);
      load8<DT>(in, in_off + d_hi, x_hi[u]);
    }
  }
  float c_lo[8], c_hi[8], s_lo[8], s_hi[8];
  load_selected<DT>(cos_t, ax, plane, tok_off, d_lo, c_lo);
  load_selected<DT>(cos_t, ax, plane, tok_off, d_hi, c_hi);
  load_selected<DT>(sin_t, ax, plane, tok_off, d_lo, s_lo);
  load_selected<DT>(sin_t, ax, plane, tok_off, d_hi, s_hi);

#pragma unroll
  for (int u = 0; u < kHeadsPerThread; ++u) {
    const int h = h0 + u;
    if (h >= n_heads) break;
    const bool is_q = h < n_q_heads;
    const int hh = is_q ? h : h - n_q_heads;
    const Strides& so = is_q ? sqo : sko;
    void* out = is_q ? q_out : k_out;
    const int64_t out_off = b * so.b + hh * so.h + s * so.s;
    float o_lo[8], o_hi[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if constexpr (!BWD) {
        // eager evaluation order of (x * cos) + (rotate_half(x) * sin): every product and the sum are
        // rounded to the storage type; rotate_half(x) = (-x_hi, x_lo)
        const float p1 = Elem<DT>::round(__fmul_rn(x_lo[u][e], c_lo[e]));
        const float p2 = Elem<DT>::round(__fmul_rn(-x_hi[u][e], s_lo[e]));
        o_lo[e] = __fadd_rn(p1, p2);
        const float p3 = Elem<DT>::round(__fmul_rn(x_hi[u][e], c_hi[e]));
        const float p4 = Elem<DT>::round(__fmul_rn(x_lo[u][e], s_hi[e]));
        o_hi[e] = __fadd_rn(p3, p4);
      } else {
        // adjoint: g*cos + rotate_half^T(g*sin), rotate_half^T(y) = (y_hi, -y_lo)
        o_lo[e] = x_lo[u][e] * c_lo[e] + x_hi[u][e] * s_hi[e];
        o_hi[e] = x_hi[u][e] * c_hi[e] - x_lo[u][e] * s_lo[e];
      }
    }
    store8<DT>(out, out_off + d_lo, o_lo);
    store8<DT>(out, out_off + d_hi, o_hi);
  }
}

// Heads whose loads are issued together in mrope_rows_kernel.
#ifndef WX_MROPE_BATCH
#define WX_MROPE_BATCH 6
#endif
constexpr int kRowsHeadBatch = WX_MROPE_BATCH;

// The chunk held by the lane `half_lanes` away (lane ^ half_lanes): the other half of the same head.
template <int L>
__device__ __forceinline__ u32x4 partner_chunk(const u32x4& v, int half_lanes) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (L == 16) {
      // rotate by 8 inside each row of 16 lanes
      r[i] = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v[i]), 0x128, 0xF, 0xF, true));
    } else {
      r[i] = static_cast<uint32_t>(__shfl_xor(static_cast<int>(v[i]), half_lanes));
    }
  }
  return r;
}

// L = lanes per head when known at compile time (16), 0 = any power of two up to 64 (runtime).
// SRC says where cos / sin come from:
//   kSrcTables     the two [3, n_tokens, head_dim] tables of the reference op;
//   kSrcPositions  no tables: `cos_t` is position_ids int64 [3, n_tokens] and `sin_t` is inv_freq fp32 [head_dim / 2].
//                  The thread evaluates cos/sin of its channels itself, the way the table builder does
//                  (vl.py:679-712): the angle is the fp32 product position * inv_freq (channels d and d + head_dim/2
//                  share a frequency), cos and sin are taken in fp32 and rounded to the storage type;
//   kSrcPacked     `cos_t` is the packed table of wx_mrope_table, uint32 [n_tokens, W] (bf16 cos | bf16 sin << 16 of
//                  the plane each channel takes): W = head_dim / 2 when channels d and d + head_dim / 2 share a plane
//                  (256 bytes per token instead of the 12 cache lines the selected channels of three planes of two
//                  tables touch), W = head_dim when they do not (one entry per channel); `sin_t` carries W as a
//                  pointer-sized integer.  bf16 only.
enum { kSrcTables = 0, kSrcPositions = 1, kSrcPacked = 2 };
template <int DT, bool BWD, int L, int SRC>
__global__ __launch_bounds__(256) void mrope_rows_kernel(
    const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ cos_t,
    const void* __restrict__ sin_t, void* __restrict__ q_out, void* __restrict__ k_out, int64_t n_tokens,
    int64_t seq, int n_q_heads, int n_kv_heads, int head_dim, Strides sq, Strides sk, Strides sqo, Strides sko,
    AxisTable ax) {
  constexpr int kEpc = 16 / Elem<DT>::kBytes;  // elements per 16-byte chunk
  const int lanes = L ? L : head_dim / kEpc;   // lanes per (token, head)
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int chunk = static_cast<int>(gid % lanes);
  int64_t token = gid / lanes;
  const bool live = token < n_tokens;
  if (!live) token = n_tokens - 1;  // lanes past the end keep taking part in the lane exchanges, and store nothing
  const int64_t b = token / seq, s = token - b * seq;
  const int d0 = chunk * kEpc;
  const bool hi = chunk >= lanes / 2;
  const int n_heads = n_q_heads + n_kv_heads;
  const u32x4* qc = reinterpret_cast<const u32x4*>(static_cast<const char*>(q) + (b * sq.b + s * sq.s + d0) * Elem<DT>::kBytes);
  const u32x4* kc = reinterpret_cast<const u32x4*>(static_cast<const char*>(k) + (b * sk.b + s * sk.s + d0) * Elem<DT>::kBytes);
  u32x4* qo = reinterpret_cast<u32x4*>(static_cast<char*>(q_out) + (b * sqo.b + s * sqo.s + d0) * Elem<DT>::kBytes);
  u32x4* ko = reinterpret_cast<u32x4*>(static_cast<char*>(k_out) + (b * sko.b + s * sko.s + d0) * Elem<DT>::kBytes);
  const int64_t hq_in = sq.h * Elem<DT>::kBytes, hk_in = sk.h * Elem<DT>::kBytes;
  const int64_t hq_out = sqo.h * Elem<DT>::kBytes, hk_out = sko.h * Elem<DT>::kBytes;

  u32x4 c_raw, s_raw;
  if constexpr (SRC == kSrcPacked) {
    static_assert(DT == WX_BF16, "the packed table holds bf16 pairs");
    const int width = static_cast<int>(reinterpret_cast<uintptr_t>(sin_t));
    const uint32_t* t = static_cast<const uint32_t*>(cos_t) + token * width + ((hi && width != head_dim) ? d0 - head_dim / 2 : d0);
    const u32x4 t0 = *reinterpret_cast<const u32x4*>(t), t1 = *reinterpret_cast<const u32x4*>(t + 4);
    c_raw = u32x4{(t0[0] & 0xffffu) | (t0[1] << 16), (t0[2] & 0xffffu) | (t0[3] << 16),
                  (t1[0] & 0xffffu) | (t1[1] << 16), (t1[2] & 0xffffu) | (t1[3] << 16)};
    s_raw = u32x4{(t0[0] >> 16) | (t0[1] & 0xffff0000u), (t0[2] >> 16) | (t0[3] & 0xffff0000u),
                  (t1[0] >> 16) | (t1[1] & 0xffff0000u), (t1[2] >> 16) | (t1[3] & 0xffff0000u)};
  } else if constexpr (SRC == kSrcPositions) {
    const int64_t pos = static_cast<const int64_t*>(cos_t)[ax.axis[d0] * n_tokens + token];
    const float* inv_freq = static_cast<const float*>(sin_t) + (hi ? d0 - head_dim / 2 : d0);
    const float pf = static_cast<float>(pos);
    float cv[kEpc], sv[kEpc];
#pragma unroll
    for (int e = 0; e < kEpc; ++e) sincosf(__fmul_rn(pf, inv_freq[e]), &sv[e], &cv[e]);
    c_raw = pack16<DT>(cv);
    s_raw = pack16<DT>(sv);
  } else {
    // selected cos / sin of my channels (regular loads: other workgroups never need them, later heads do not
    // either, but the three position planes are small next to q)
    const int64_t tab_off = (ax.axis[d0] * (n_tokens * head_dim) + token * head_dim + d0) * Elem<DT>::kBytes;
    c_raw = *reinterpret_cast<const u32x4*>(static_cast<const char*>(cos_t) + tab_off);
    s_raw = *reinterpret_cast<const u32x4*>(static_cast<const char*>(sin_t) + tab_off);
  }
  if constexpr (BWD) s_raw = partner_chunk<L>(s_raw, lanes / 2);  // the adjoint multiplies by the partner's sin
  float c[kEpc], sn[kEpc];
  unpack16<DT>(c_raw, c);
  unpack16<DT>(s_raw, sn);
  // forward: out = x*cos + rotate_half(x)*sin with rotate_half(x) = (-x_hi, x_lo): the low half takes -partner
  // adjoint: out = g*cos + rotate_half^T(g*sin) with rotate_half^T(y) = (y_hi, -y_lo): the high half takes -partner
  const float sign = (hi != BWD) ? 1.0f : -1.0f;
#pragma unroll
  for (int e = 0; e < kEpc; ++e) sn[e] *= sign;  // exact

  for (int h0 = 0; h0 < n_heads; h0 += kRowsHeadBatch) {
    u32x4 raw[kRowsHeadBatch];
#pragma unroll
    for (int u = 0; u < kRowsHeadBatch; ++u) {
      const int h = h0 + u;
      if (h < n_heads) {
        const u32x4* src = h < n_q_heads
            ? reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(qc) + h * hq_in)
            : reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(kc) + (h - n_q_heads) * hk_in);
        raw[u] = __builtin_nontemporal_load(src);
      }
    }
#pragma unroll
    for (int u = 0; u < kRowsHeadBatch; ++u) {
      const int h = h0 + u;
      if (h < n_heads) {  // uniform over the workgroup
        const u32x4 other = partner_chunk<L>(raw[u], lanes / 2);
        float x[kEpc], xp[kEpc], o[kEpc];
        unpack16<DT>(raw[u], x);
        unpack16<DT>(other, xp);
#pragma unroll
        for (int e = 0; e < kEpc; ++e) {
          if constexpr (!BWD) {
            // eager evaluation order of (x * cos) + (rotate_half(x) * sin): every product and the sum are rounded
            // to the storage type (the sum by the final pack)
            const float p1 = Elem<DT>::round(__fmul_rn(x[e], c[e]));
            const float p2 = Elem<DT>::round(__fmul_rn(xp[e], sn[e]));
            o[e] = __fadd_rn(p1, p2);
          } else {
            o[e] = __fadd_rn(__fmul_rn(x[e], c[e]), __fmul_rn(xp[e], sn[e]));
          }
        }
        if (live) {
          u32x4* dst = h < n_q_heads ? reinterpret_cast<u32x4*>(reinterpret_cast<char*>(qo) + h * hq_out)
                                     : reinterpret_cast<u32x4*>(reinterpret_cast<char*>(ko) + (h - n_q_heads) * hk_out);
          __builtin_nontemporal_store(pack16<DT>(o), dst);
        }
      }
    }
  }
}

int build_axis_table(const int sec[3], int head_dim, int layout, AxisTable& ax) {
  int d = 0;
  auto put = [&](int axis, int n) {
    for (int i = 0; i < n && d < kMaxHeadDim; ++i) ax.axis[d++] = static_cast<uint8_t>(axis);
  };
  if (layout == WX_MROPE_HF) {
    for (int rep = 0; rep < 2; ++rep)
      for (int a = 0; a < 3; ++a) put(a, sec[a]);
  } else if (layout == WX_MROPE_CSRC) {
    put(0, 2 * sec[0]);
    put(1, 2 * sec[1]);
    while (d < head_dim) put(2, 1);  // csrc/rope.cu:104-117: everything past s0+s1 is the w plane
  } else {
    return fail(WX_ERR_INVALID_ARGUMENT, "mrope: bad layout %d", layout);
  }
  if (d != head_dim)
    return fail(WX_ERR_INVALID_ARGUMENT, "mrope: mrope_section [%d,%d,%d] covers %d channels, head_dim is %d", sec[0],
                sec[1], sec[2], d, head_dim);
  for (int c = 0; c < head_dim / 8; ++c) {
    bool same = true;
    for (int e = 1; e < 8; ++e) same = same && ax.axis[8 * c + e] == ax.axis[8 * c];
    ax.uniform[c] = same;
  }
  return WX_OK;
}

// Entries per token of the packed table: head_dim / 2 when every channel d shares its position plane with channel
// d + head_dim / 2 (the PyTorch path's layout, vl.py:763-769: one entry serves both), head_dim otherwise (the CUDA
// kernel's layout, csrc/rope.cu:104-117: one entry per channel).
int packed_table_width(const AxisTable& ax, int head_dim) {
  for (int d = 0; d < head_dim / 2; ++d)
    if (ax.axis[d] != ax.axis[d + head_dim / 2]) return head_dim;
  return head_dim / 2;
}

// SRC: what cos_t / sin_t carry (see mrope_rows_kernel)
template <bool BWD, int SRC = kSrcTables>
int launch(const void* q, const void* k, const void* cos_t, const void* sin_t, void* q_out, void* k_out,
           int64_t batch, int64_t seq, int n_q, int n_kv, int head_dim, const int64_t* sq, const int64_t* sk,
           const int64_t* sqo, const int64_t* sko, const int sec[3], int layout, int dtype, wx_stream_t stream) {
  const char* who = SRC == kSrcPositions ? (BWD ? "wx_mrope_apply_positions(backward)" : "wx_mrope_apply_positions")
                    : SRC == kSrcPacked  ? (BWD ? "wx_mrope_apply_packed(backward)" : "wx_mrope_apply_packed")
                                         : (BWD ? "wx_mrope_apply_bwd" : "wx_mrope_apply");
  if (batch < 0 || seq < 0 || n_q < 0 || n_kv < 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: negative size", who);
  if (head_dim <= 0 || head_dim % 16 != 0 || head_dim > kMaxHeadDim)
    return fail(WX_ERR_UNSUPPORTED, "%s: head_dim %d must be a multiple of 16 and <= %d", who, head_dim, kMaxHeadDim);
  if (!sq || !sk || !sqo || !sko || !sec) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null stride/section", who);
  const int64_t n_tokens = batch * seq;
  if (n_tokens == 0 || n_q + n_kv == 0) return WX_OK;
  if (!cos_t || (SRC != kSrcPacked && !sin_t) || (n_q && (!q || !q_out)) || (n_kv && (!k || !k_out)))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if (SRC == kSrcPacked && dtype != WX_BF16) return fail(WX_ERR_UNSUPPORTED, "%s: the packed table is bf16", who);
  const int align = dtype == WX_F32 ? 4 : 8;  // elements per 16 bytes
  const int64_t* all[4] = {sq, sk, sqo, sko};
  for (auto* st : all)
    for (int i = 0; i < 3; ++i)
      if (st[i] % align != 0) return fail(WX_ERR_UNSUPPORTED, "%s: strides must keep rows 16-byte aligned", who);
  AxisTable ax{};
  if (int rc = build_axis_table(sec, head_dim, layout, ax)) return rc;
  if constexpr (SRC == kSrcPacked) {
    // the table's width follows from the layout exactly as in wx_mrope_table; it travels in the unused `sin_t` slot
    sin_t = reinterpret_cast<const void*>(static_cast<uintptr_t>(packed_table_width(ax, head_dim)));
  }
  const Strides a{sq[0], sq[1], sq[2]}, b{sk[0], sk[1], sk[2]}, c{sqo[0], sqo[1], sqo[2]}, d{sko[0], sko[1], sko[2]};
  hipStream_t s = as_stream(stream);
  // Row form: 16-byte chunks per head must be a power of two that divides the workgroup, and no section boundary
  // may cut through a chunk.
  const int epc = dtype == WX_F32 ? 4 : 8;
  const int lanes = head_dim / epc;
  bool rows_ok = lanes >= 2 && lanes <= 64 && (lanes & (lanes - 1)) == 0;
  for (int cidx = 0; cidx < head_dim / 8 && rows_ok; ++cidx) rows_ok = ax.uniform[cidx] != 0;
  if (rows_ok) {
    const int64_t threads = n_tokens * lanes;
    if ((threads + 255) / 256 > 0x7fffffffll) return fail(WX_ERR_UNSUPPORTED, "%s: too many tokens", who);
    const dim3 grid(static_cast<unsigned>((threads + 255) / 256)), block(256);
#define WX_LAUNCH_ROWS(DT, L)                                                                                       \
  hipLaunchKernelGGL((mrope_rows_kernel<DT, BWD, L, SRC>), grid, block, 0, s, q, k, cos_t, sin_t, q_out, k_out, n_tokens, \
                     seq, n_q, n_kv, head_dim, a, b, c, d, ax)
    if constexpr (SRC == kSrcPacked) {
      if (lanes == 16) WX_LAUNCH_ROWS(WX_BF16, 16); else WX_LAUNCH_ROWS(WX_BF16, 0);
    } else {
      switch (dtype) {
        case WX_F32: WX_LAUNCH_ROWS(WX_F32, 0); break;
        case WX_F16: if (lanes == 16) WX_LAUNCH_ROWS(WX_F16, 16); else WX_LAUNCH_ROWS(WX_F16, 0); break;
        case WX_BF16: if (lanes == 16) WX_LAUNCH_ROWS(WX_BF16, 16); else WX_LAUNCH_ROWS(WX_BF16, 0); break;
        default: return fail(WX_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
      }
    }
#undef WX_LAUNCH_ROWS
    return check_launch(who);
  }
  if constexpr (SRC != kSrcTables) {
    return fail(WX_ERR_UNSUPPORTED,
                "%s: needs a head of 2..64 16-byte chunks (a power of two) and sections that end on chunk boundaries; "
                "build the cos/sin tables and call wx_mrope_apply instead", who);
  } else {
  // grid.x walks (token, rotation group); grid.y walks groups of kHeadsPerThread heads
  const int groups = head_dim / 16;
  const int head_groups = (n_q + n_kv + kHeadsPerThread - 1) / kHeadsPerThread;
  const int64_t threads = n_tokens * groups;
  if ((threads + 255) / 256 > 0x7fffffffll) return fail(WX_ERR_UNSUPPORTED, "%s: too many tokens", who);
  const dim3 grid(static_cast<unsigned>((threads + 255) / 256), static_cast<unsigned>(head_groups)), block(256);
#define WX_LAUNCH(DT)                                                                                             \
  hipLaunchKernelGGL((mrope_kernel<DT, BWD>), grid, block, 0, s, q, k, cos_t, sin_t, q_out, k_out, n_tokens, seq, \
                     n_q, n_kv, head_dim, a, b, c, d, ax)
  switch (dtype) {
    case WX_F32: WX_LAUNCH(WX_F32); break;
    case WX_F16: WX_LAUNCH(WX_F16); break;
    case WX_BF16: WX_LAUNCH(WX_BF16); break;
    default: return fail(WX_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  }
#undef WX_LAUNCH
  return check_launch(who);
  }
}

// Packed rotary table for the projection kernel that rotates q and k in its epilogue and for the packed form of the
// apply kernel: entry [token][d], d < width, holds cos (low half) and sin (high half) of
// position[plane(d)] * inv_freq[d mod half], rounded to bf16 like the table builder's output (vl.py:679-712).
// width = half when channels d and d + half take the same plane (the PyTorch path's layout, vl.py:763-769), else
// 2 * half, one entry per channel (the CUDA kernel's layout, csrc/rope.cu:104-117).
__global__ __launch_bounds__(256) void mrope_table_kernel(const int64_t* __restrict__ pos,
                                                          const float* __restrict__ inv_freq,
                                                          uint32_t* __restrict__ out, int64_t n_tokens, int half,
                                                          int width, AxisTable ax) {
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid >= n_tokens * width) return;
  const int64_t token = gid / width;
  const int d = static_cast<int>(gid - token * width);
  const float pf = static_cast<float>(pos[ax.axis[d] * n_tokens + token]);
  float sv, cv;
  sincosf(__fmul_rn(pf, inv_freq[d >= half ? d - half : d]), &sv, &cv);
  out[gid] = f32_to_bf16_bits(cv) | (f32_to_bf16_bits(sv) << 16);
}

}  // namespace
}  // namespace wx

extern "C" int wx_mrope_apply(const void* q, const void* k, const void* cos, const void* sin, void* q_out,
                              void* k_out, int64_t batch, int64_t seq, int n_q_heads, int n_kv_heads, int head_dim,
                              const int64_t q_strides[3], const int64_t k_strides[3], const int64_t qo_strides[3],
                              const int64_t ko_strides[3], const int mrope_section[3], int layout, int dtype,
                              wx_stream_t stream) {
  return wx::launch<false>(q, k, cos, sin, q_out, k_out, batch, seq, n_q_heads, n_kv_heads, head_dim, q_strides,
                           k_strides, qo_strides, ko_strides, mrope_section, layout, dtype, stream);
}

extern "C" int wx_mrope_apply_bwd(const void* gq_out, const void* gk_out, const void* cos, const void* sin, void* gq,
                                  void* gk, int64_t batch, int64_t seq, int n_q_heads, int n_kv_heads, int head_dim,
                                  const int64_t gqo_strides[3], const int64_t gko_strides[3],
                                  const int64_t gq_strides[3], const int64_t gk_strides[3],
                                  const int mrope_section[3], int layout, int dtype, wx_stream_t stream) {
  return wx::launch<true>(gq_out, gk_out, cos, sin, gq, gk, batch, seq, n_q_heads, n_kv_heads, head_dim, gqo_strides,
                          gko_strides, gq_strides, gk_strides, mrope_section, layout, dtype, stream);
}

extern "C" int wx_mrope_apply_positions(const void* q, const void* k, const int64_t* position_ids,
                                        const float* inv_freq, void* q_out, void* k_out, int64_t batch, int64_t seq,
                                        int n_q_heads, int n_kv_heads, int head_dim, const int64_t q_strides[3],
                                        const int64_t k_strides[3], const int64_t qo_strides[3],
                                        const int64_t ko_strides[3], const int mrope_section[3], int layout,
                                        int dtype, int backward, wx_stream_t stream) {
  if (backward)
    return wx::launch<true, wx::kSrcPositions>(q, k, position_ids, inv_freq, q_out, k_out, batch, seq, n_q_heads, n_kv_heads,
                                  head_dim, q_strides, k_strides, qo_strides, ko_strides, mrope_section, layout, dtype,
                                  stream);
  return wx::launch<false, wx::kSrcPositions>(q, k, position_ids, inv_freq, q_out, k_out, batch, seq, n_q_heads, n_kv_heads,
                                 head_dim, q_strides, k_strides, qo_strides, ko_strides, mrope_section, layout, dtype,
                                 stream);
}

extern "C" int wx_mrope_apply_packed(const void* q, const void* k, const uint32_t* table, void* q_out, void* k_out,
                                     int64_t batch, int64_t seq, int n_q_heads, int n_kv_heads, int head_dim,
                                     const int64_t q_strides[3], const int64_t k_strides[3],
                                     const int64_t qo_strides[3], const int64_t ko_strides[3],
                                     const int mrope_section[3], int layout, int dtype, int backward,
                                     wx_stream_t stream) {
  if (reinterpret_cast<uintptr_t>(table) & 15)
    return wx::fail(WX_ERR_INVALID_ARGUMENT, "wx_mrope_apply_packed: the table must be 16-byte aligned");
  if (backward)
    return wx::launch<true, wx::kSrcPacked>(q, k, table, nullptr, q_out, k_out, batch, seq, n_q_heads, n_kv_heads,
                                            head_dim, q_strides, k_strides, qo_strides, ko_strides, mrope_section,
                                            layout, dtype, stream);
  return wx::launch<false, wx::kSrcPacked>(q, k, table, nullptr, q_out, k_out, batch, seq, n_q_heads, n_kv_heads,
                                           head_dim, q_strides, k_strides, qo_strides, ko_strides, mrope_section,
                                           layout, dtype, stream);
}

extern "C" int wx_mrope_table(const int64_t* position_ids, const float* inv_freq, int64_t batch, int64_t seq,
                              int head_dim, const int mrope_section[3], int layout, uint32_t* table,
                              wx_stream_t stream) {
  using namespace wx;
  const char* who = "wx_mrope_table";
  if (batch < 0 || seq < 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: negative size", who);
  if (head_dim <= 0 || head_dim % 16 != 0 || head_dim > kMaxHeadDim)
    return fail(WX_ERR_UNSUPPORTED, "%s: head_dim %d must be a multiple of 16 and <= %d", who, head_dim, kMaxHeadDim);
  if (!mrope_section) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null section", who);
  AxisTable ax{};
  if (int rc = build_axis_table(mrope_section, head_dim, layout, ax)) return rc;
  const int half = head_dim / 2;
  const int width = packed_table_width(ax, head_dim);
  const int64_t n = batch * seq * width;
  if (n == 0) return WX_OK;
  if (!position_ids || !inv_freq || !table) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((n + 255) / 256 > 0x7fffffffll) return fail(WX_ERR_UNSUPPORTED, "%s: too many tokens", who);
  hipLaunchKernelGGL(mrope_table_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, as_stream(stream),
                     position_ids, inv_freq, table, batch * seq, half, width, ax);
  return check_launch(who);
}

extern "C" int wx_mrope_table_width(int head_dim, const int mrope_section[3], int layout) {
  using namespace wx;
  const char* who = "wx_mrope_table_width";
  if (head_dim <= 0 || head_dim % 16 != 0 || head_dim > kMaxHeadDim)
    return fail(WX_ERR_UNSUPPORTED, "%s: head_dim %d must be a multiple of 16 and <= %d", who, head_dim, kMaxHeadDim);
  if (!mrope_section) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null section", who);
  AxisTable ax{};
  if (int rc = build_axis_table(mrope_section, head_dim, layout, ax)) return rc;
  return packed_table_width(ax, head_dim);
}
