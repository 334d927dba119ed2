// Dual asymmetric grouped GEMM and the fused dual-expert SwiGLU FFN for gfx950 (bf16 MFMA, fp32 accumulate).
//
// One persistent launch covers the tiles of BOTH experts: the grid is one workgroup per CU, the tile list
// is derived on the device from the per-expert row counts (host values or the partition's device-side
// expert_offsets), and a tile id -> (expert, tile_m, tile_n) map keeps the 32 tiles that run concurrently
// on one XCD inside a compact patch of the output so they share A/B slabs through that XCD's L2.
// A skewed pair (thousands of VL rows, tens of action rows, or an empty group) is just a longer or
// shorter tile list; no CU waits for "its" expert.
//
// Workgroup tile 256 x 256 x 64, 8 wavefronts as 2 (M) x 4 (N), wave tile 128 x 64 = 4 x 2 MFMA
// 32x32x16 accumulators.  Operands are K-contiguous ([m,k] activations, [n,k] nn.Linear weights), so both
// fragments are 16-byte LDS reads.  Global -> LDS goes through buffer loads that write LDS directly
// (no VGPR staging), double buffered, one barrier per K step; rows past the end of a matrix read as zero
// through the buffer bounds check.  LDS rows are 128 bytes (64 bf16); the 16-byte chunk c of row r is
// stored at slot c ^ ((r >> 1) & 7) so that the 16 rows a quarter-wave reads land on distinct banks.
//
// SwiGLU mode: the B tile is 128 gate rows + 128 up rows of the same intermediate columns, so gate and
// up accumulators of one output element sit in the same lane and register index; the epilogue applies
// silu(g) * u with eager bf16 rounding and writes the 256 x 128 intermediate tile.
#include "common.h"

namespace wx {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 512;
constexpr int kRowBytes = BK * 2;              // 128 bytes of K per LDS row
constexpr int kTileBytes = BM * kRowBytes;     // 32 KiB per operand per stage
constexpr int kXcds = 8;
constexpr int kGroupM = 8;                     // tile rows per patch in the tile order

struct Group {
  const __bf16* a;    // [m, k] row-major, leading dimension lda
  const __bf16* b0;   // [n, k] row-major (SwiGLU: gate)
  const __bf16* b1;   // SwiGLU: up; otherwise unused
  __bf16* c;          // [m, n] row-major, leading dimension ldc
  int m, n, k;
  int lda, ldb, ldc;
};

struct Params {
  Group g[2];
  const int32_t* offsets;  // device int32[3]: rows of expert e are [offsets[e], offsets[e+1]); or null
};

#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// Buffer descriptor for `bytes` readable bytes at `base`.  Both are wave-uniform by construction; passing them
// through readfirstlane pins the descriptor to scalar registers.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t v = reinterpret_cast<uint64_t>(base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  void* p = reinterpret_cast<void*>((static_cast<uint64_t>(hi) << 32) | lo);
  return __builtin_amdgcn_make_buffer_rsrc(p, 0, static_cast<int>(__builtin_amdgcn_readfirstlane(bytes)), 0x00020000);
}

struct TileCoord {
  int group, tm, tn;
};

// Linear tile id -> coordinates.  Ids are first spread so that each XCD (workgroup id mod 8) walks its own
// contiguous range of "virtual" ids; virtual ids then sweep patches of kGroupM tile rows column by column.
__device__ __forceinline__ bool map_tile(int64_t t, int64_t total, const int* tiles_m, const int* tiles_n,
                                         TileCoord& tc) {
  const int64_t per = (total + kXcds - 1) / kXcds;
  int64_t v = (t % kXcds) * per + t / kXcds;
  if (v >= total) return false;
  int g = 0;
  const int64_t c0 = static_cast<int64_t>(tiles_m[0]) * tiles_n[0];
  if (v >= c0) { g = 1; v -= c0; }
  const int tmn = g ? tiles_m[1] : tiles_m[0], tnn = g ? tiles_n[1] : tiles_n[0];
  const int64_t patch = static_cast<int64_t>(kGroupM) * tnn;
  const int first_m = static_cast<int>(v / patch) * kGroupM;
  const int rows = tmn - first_m < kGroupM ? tmn - first_m : kGroupM;
  const int64_t in_patch = v % patch;
  tc.group = g;
  tc.tm = first_m + static_cast<int>(in_patch % rows);
  tc.tn = static_cast<int>(in_patch / rows);
  return true;
}

template <bool SWIGLU>
__global__ __launch_bounds__(kThreads, 1) void dual_gemm_kernel(Params p) {
  __shared__ __attribute__((aligned(1024))) unsigned char s_a0[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_b0[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_a1[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_b1[kTileBytes];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps descriptors and LDS bases scalar
  const int wm = wave >> 2, wn = wave & 3;
  const int l32 = lane & 31, lhi = lane >> 5;

  // ---- problem table (uniform) ------------------------------------------------------------------
  // (kept as two named structs, selected per tile, so everything stays in scalar registers)
  Group g0 = p.g[0], g1 = p.g[1];
  if (p.offsets != nullptr) {
    const int o0 = p.offsets[0], o1 = p.offsets[1], o2 = p.offsets[2];
    g0.m = o1 - o0;
    g1.m = o2 - o1;
    g0.a += static_cast<int64_t>(o0) * g0.lda;
    g0.c += static_cast<int64_t>(o0) * g0.ldc;
    g1.a = g0.a + static_cast<int64_t>(g0.m) * g0.lda;
    g1.c = g0.c + static_cast<int64_t>(g0.m) * g0.ldc;
  }
  constexpr int kTileN = SWIGLU ? BN / 2 : BN;  // output columns per tile
  int tiles_m[2], tiles_n[2];
  tiles_m[0] = (g0.m + BM - 1) / BM;
  tiles_n[0] = (g0.n + kTileN - 1) / kTileN;
  if (g0.m <= 0 || g0.n <= 0) tiles_m[0] = tiles_n[0] = 0;
  tiles_m[1] = (g1.m + BM - 1) / BM;
  tiles_n[1] = (g1.n + kTileN - 1) / kTileN;
  if (g1.m <= 0 || g1.n <= 0) tiles_m[1] = tiles_n[1] = 0;
  const int64_t total = static_cast<int64_t>(tiles_m[0]) * tiles_n[0] + static_cast<int64_t>(tiles_m[1]) * tiles_n[1];
  const int64_t padded = (total + kXcds - 1) / kXcds * kXcds;

  // ---- per-lane constants -----------------------------------------------------------------------
  // loader: instruction i of this wave fills LDS rows [wave*32 + 8i, +8); lane -> (row lane/8, slot lane%8)
  const int ld_row0 = wave * 32 + (lane >> 3);
  int ld_chunk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = ld_row0 + 8 * i;
    ld_chunk[i] = (lane & 7) ^ ((row >> 1) & 7);
  }
  // fragment reads: row = base + l32, chunk kc = 2*kk + lhi stored at slot kc ^ ((l32 >> 1) & 7)
  const int sw = (l32 >> 1) & 7;
  int frag_off[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) frag_off[kk] = ((2 * kk + lhi) ^ sw) << 4;
  const int a_row_off = (wm * 128 + l32) * kRowBytes;
  const int b_row_off0 = (SWIGLU ? wn * 32 + l32 : wn * 64 + l32) * kRowBytes;
  const int b_row_off1 = (SWIGLU ? 128 + wn * 32 + l32 : wn * 64 + 32 + l32) * kRowBytes;

  // ---- per-tile state ------------------------------------------------------------------------------
  struct Loader {   // where this thread's eight 16-byte loads per K step come from
    const __bf16 *a_base, *b_base;
    uint32_t a_bytes, b_bytes;
    uint32_t voff_a[4], voff_b[4];
    int K, nk;
  };
  struct Store {    // where the finished tile goes
    __bf16* c_base;
    int rows, cols_left, ldc;  // valid rows / columns from the tile origin
  };

  auto setup = [&](const TileCoord& tc, Loader& L, Store& S) {
    const Group G = tc.group ? g1 : g0;
    const int row0 = tc.tm * BM, col0 = tc.tn * kTileN;
    const int rows_a = G.m - row0 < BM ? G.m - row0 : BM;
    const int rows_b = G.n - col0 < kTileN ? G.n - col0 : kTileN;
    L.K = G.k;
    L.nk = (G.k + BK - 1) / BK;
    L.a_base = G.a + static_cast<int64_t>(row0) * G.lda;
    const bool up_half = SWIGLU && wave >= 4;
    L.b_base = (up_half ? G.b1 : G.b0) + static_cast<int64_t>(col0) * G.ldb;
    L.a_bytes = static_cast<uint32_t>(rows_a) * G.lda * 2u;
    L.b_bytes = static_cast<uint32_t>(rows_b) * G.ldb * 2u;
    const int b_ld_row0 = SWIGLU ? (wave & 3) * 32 + (lane >> 3) : ld_row0;  // row inside the gate / up half
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      L.voff_a[i] = static_cast<uint32_t>(ld_row0 + 8 * i) * G.lda * 2u + ld_chunk[i] * 16u;
      L.voff_b[i] = static_cast<uint32_t>(b_ld_row0 + 8 * i) * G.ldb * 2u + ld_chunk[i] * 16u;
    }
    S.c_base = G.c + static_cast<int64_t>(row0) * G.ldc + col0;
    S.rows = rows_a;
    S.cols_left = G.n - col0;
    S.ldc = G.ldc;
  };

  // One K step of global -> LDS for this wave: rows [wave*32, +32) of the A tile and of the B tile.
  auto issue = [&](const Loader& L, int ks, unsigned char* sa, unsigned char* sb) {
    const int k0 = ks * BK;
    // advancing the base keeps the absolute end of the readable range: rows past the matrix and, through the
    // per-lane select below, K chunks past the row end read as zero
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(L.a_base + k0, L.a_bytes - 2u * k0);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(L.b_base + k0, L.b_bytes - 2u * k0);
    const bool k_tail = k0 + BK > L.K;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t va = L.voff_a[i], vb = L.voff_b[i];
      if (k_tail && k0 + ld_chunk[i] * 8 >= L.K) va = vb = 0x80000000u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, LDS_PTR(sa + (wave * 32 + 8 * i) * kRowBytes), 16, va, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, LDS_PTR(sb + (wave * 32 + 8 * i) * kRowBytes), 16, vb, 0, 0, 0);
    }
  };

  f32x16 acc[4][2];
  bf16x8 fa[2][4], fb[2][2];  // two fragment sets: one feeds the MFMAs while the other is being read from LDS

  auto read_frags = [&](const unsigned char* sa, const unsigned char* sb, int kk, int set) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      fa[set][i] = *reinterpret_cast<const bf16x8*>(sa + a_row_off + i * 32 * kRowBytes + frag_off[kk]);
    fb[set][0] = *reinterpret_cast<const bf16x8*>(sb + b_row_off0 + frag_off[kk]);
    fb[set][1] = *reinterpret_cast<const bf16x8*>(sb + b_row_off1 + frag_off[kk]);
  };
  auto mma = [&](int set) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
  };
  // scheduling hints: interleave the six LDS reads of the next fragment set with the eight MFMAs of this one
  auto interleave_reads = [&]() {
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
  };

  // One K step.  On entry fragment set 0 holds kk = 0 of the current stage.  The barrier sits before the last
  // quarter: by then every wave has its kk = 3 fragments in registers, so the current stage can be refilled
  // (K step ks + 2) right after it, and the next stage -- issued a whole K step earlier -- is complete.
  auto k_step = [&](const Loader& L, int ks, unsigned char* sa_cur, unsigned char* sb_cur, unsigned char* sa_nxt,
                    unsigned char* sb_nxt) {
    read_frags(sa_cur, sb_cur, 1, 1);
    mma(0);
    interleave_reads();
    read_frags(sa_cur, sb_cur, 2, 0);
    mma(1);
    interleave_reads();
    read_frags(sa_cur, sb_cur, 3, 1);
    mma(0);
    interleave_reads();
    if (ks + 1 < L.nk) {
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): my loads for ks+1 landed, my LDS reads returned
      __syncthreads();
      if (ks + 2 < L.nk) issue(L, ks + 2, sa_cur, sb_cur);
      read_frags(sa_nxt, sb_nxt, 0, 0);
    }
    mma(1);
  };

  auto epilogue = [&](const Store& S) {
    // accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 block
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
        if (row >= S.rows) continue;
        __bf16* c_row = S.c_base + static_cast<int64_t>(row) * S.ldc;
        if constexpr (SWIGLU) {
          const int col = wn * 32 + l32;
          if (col < S.cols_left) {
            // eager bf16 evaluation of act_fn(gate) * up (act.py:80-82): gate, up, silu(gate) and the product are
            // each rounded to bf16
            const float g = round_bf16(acc[i][0][r]);
            const float u = round_bf16(acc[i][1][r]);
            const float sg = round_bf16(g / (1.0f + expf(-g)));
            c_row[col] = static_cast<__bf16>(sg * u);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int col = wn * 64 + j * 32 + l32;
            if (col < S.cols_left) c_row[col] = static_cast<__bf16>(acc[i][j][r]);
          }
        }
      }
    }
  };

  // first two K steps of a tile go out together; later ones are issued from inside k_step
  auto prologue = [&](const Loader& L) {
    issue(L, 0, s_a0, s_b0);
    if (L.nk > 1) issue(L, 1, s_a1, s_b1);
  };

  // ---- persistent tile loop -----------------------------------------------------------------------
  int64_t t = blockIdx.x;
  TileCoord tc;
  bool have = false;
  for (; t < padded && !have; t += have ? 0 : gridDim.x) have = map_tile(t, total, tiles_m, tiles_n, tc);
  if (!have) return;
  Loader L;
  Store S;
  setup(tc, L, S);
  prologue(L);

  while (true) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // stage 0 (K step 0) must be complete; K step 1 may still be in flight (8 loads per wave per K step)
    if (L.nk > 1) __builtin_amdgcn_s_waitcnt(0x0F78); else __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    read_frags(s_a0, s_b0, 0, 0);
    for (int ks = 0; ks < L.nk; ks += 2) {
      k_step(L, ks, s_a0, s_b0, s_a1, s_b1);
      if (ks + 1 < L.nk) k_step(L, ks + 1, s_a1, s_b1, s_a0, s_b0);
    }

    // next tile: its first loads fly while this tile's results are stored
    TileCoord tn;
    bool more = false;
    for (t += gridDim.x; t < padded && !more; t += more ? 0 : gridDim.x) more = map_tile(t, total, tiles_m, tiles_n, tn);
    const Store done = S;
    __syncthreads();  // every wave holds its last fragments in registers: both stages are free
    if (more) {
      setup(tn, L, S);
      prologue(L);
    }
    epilogue(done);
    if (!more) break;
  }
}

// ---- generic fallback: any transpose combination, any k; one thread per output element pair -----------
// Used for the layouts the MFMA kernel does not read in place (trans_a, or weights stored [k, n]).
__global__ __launch_bounds__(256) void dual_gemm_reference_layout_kernel(Params p, int trans_a, int trans_b) {
  __shared__ float s_a[32][33];
  __shared__ float s_b[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8 threads, 32 x 32 output tile
  for (int e = 0; e < 2; ++e) {
    const Group& G = p.g[e];
    if (G.m <= 0 || G.n <= 0) continue;
    const int tiles_n = (G.n + 31) / 32, tiles_m = (G.m + 31) / 32;
    for (int64_t t = blockIdx.x; t < static_cast<int64_t>(tiles_m) * tiles_n; t += gridDim.x) {
      const int row0 = static_cast<int>(t / tiles_n) * 32, col0 = static_cast<int>(t % tiles_n) * 32;
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
      for (int k0 = 0; k0 < G.k; k0 += 32) {
        for (int r = ty; r < 32; r += 8) {
          const int m = row0 + r, n = col0 + r, k = k0 + tx;
          float av = 0.f, bv = 0.f;
          if (k < G.k && m < G.m)
            av = static_cast<float>(trans_a ? G.a[static_cast<int64_t>(k) * G.lda + m] : G.a[static_cast<int64_t>(m) * G.lda + k]);
          if (k < G.k && n < G.n)
            bv = static_cast<float>(trans_b ? G.b0[static_cast<int64_t>(n) * G.ldb + k] : G.b0[static_cast<int64_t>(k) * G.ldb + n]);
          s_a[r][tx] = av;  // s_a[m][k]
          s_b[r][tx] = bv;  // s_b[n][k]
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 32; ++kk) {
          const float bv = s_b[tx][kk];
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[q] += s_a[ty + 8 * q][kk] * bv;
        }
        __syncthreads();
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = row0 + ty + 8 * q, n = col0 + tx;
        if (m < G.m && n < G.n) G.c[static_cast<int64_t>(m) * G.ldc + n] = static_cast<__bf16>(acc[q]);
      }
    }
  }
}

int check_dims(const char* who, int64_t m, int64_t n, int64_t k) {
  if (m < 0 || n < 0 || k < 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: negative dimension", who);
  if (m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: dimension exceeds int32", who);
  if (n % 8 != 0 || k % 8 != 0)
    return fail(WX_ERR_UNSUPPORTED, "%s: n (%lld) and k (%lld) must be multiples of 8", who, static_cast<long long>(n),
                static_cast<long long>(k));
  // 256 rows of one operand must stay addressable through a 31-bit buffer offset
  if (k * 2 * 256 >= (1ll << 31) || n * 2 * 256 >= (1ll << 31)) return fail(WX_ERR_UNSUPPORTED, "%s: row too long", who);
  return WX_OK;
}

template <bool SWIGLU>
int launch_mfma(const Params& p, hipStream_t s, const char* who) {
  hipLaunchKernelGGL(dual_gemm_kernel<SWIGLU>, dim3(device_cu_count()), dim3(kThreads), 0, s, p);
  return check_launch(who);
}

}  // namespace
}  // namespace wx

using namespace wx;

extern "C" int wx_dual_gemm(const void* in0, const void* in1, const void* w0, const void* w1, void* out0, void* out1,
                            int64_t m0, int64_t n0, int64_t k0, int64_t m1, int64_t n1, int64_t k1, int trans_a,
                            int trans_b, wx_stream_t stream) {
  if (int rc = check_dims("wx_dual_gemm", m0, n0, k0)) return rc;
  if (int rc = check_dims("wx_dual_gemm", m1, n1, k1)) return rc;
  const void* ptrs[2][3] = {{in0, w0, out0}, {in1, w1, out1}};
  const int64_t dims[2][3] = {{m0, n0, k0}, {m1, n1, k1}};
  Params p{};
  for (int e = 0; e < 2; ++e) {
    const int64_t m = dims[e][0], n = dims[e][1], k = dims[e][2];
    if (m > 0 && n > 0 && (!ptrs[e][2] || (k > 0 && (!ptrs[e][0] || !ptrs[e][1]))))
      return fail(WX_ERR_INVALID_ARGUMENT, "wx_dual_gemm: null pointer for expert %d", e);
    for (int q = 0; q < 3; ++q)
      if (reinterpret_cast<uintptr_t>(ptrs[e][q]) & 15)
        return fail(WX_ERR_INVALID_ARGUMENT, "wx_dual_gemm: buffers must be 16-byte aligned");
    if (trans_a && m % 8 != 0) return fail(WX_ERR_UNSUPPORTED, "wx_dual_gemm: trans_a needs m to be a multiple of 8");
    Group& g = p.g[e];
    g.a = static_cast<const __bf16*>(ptrs[e][0]);
    g.b0 = static_cast<const __bf16*>(ptrs[e][1]);
    g.b1 = nullptr;
    g.c = static_cast<__bf16*>(const_cast<void*>(ptrs[e][2]));
    g.m = static_cast<int>(m); g.n = static_cast<int>(n); g.k = static_cast<int>(k);
    g.lda = static_cast<int>(trans_a ? m : k);
    g.ldb = static_cast<int>(trans_b ? k : n);
    g.ldc = static_cast<int>(n);
  }
  p.offsets = nullptr;
  if ((m0 == 0 || n0 == 0) && (m1 == 0 || n1 == 0)) return WX_OK;
  hipStream_t s = as_stream(stream);
  if (!trans_a && trans_b) return launch_mfma<false>(p, s, "dual_gemm_kernel");
  hipLaunchKernelGGL(dual_gemm_reference_layout_kernel, dim3(device_cu_count() * 4), dim3(256), 0, s, p, trans_a, trans_b);
  return check_launch("dual_gemm_reference_layout_kernel");
}

namespace {

struct FfnArgs {
  const void *x, *gate[2], *up[2], *down[2];
  void *out, *hmid;
  const int32_t* offsets;
  int64_t rows, hidden, inter[2];
};

int check_ffn(const char* who, const FfnArgs& a, bool need_gate_up, bool need_down) {
  if (int rc = check_dims(who, a.rows, a.inter[0], a.hidden)) return rc;
  if (int rc = check_dims(who, a.rows, a.hidden, a.inter[1])) return rc;
  if (a.rows == 0) return WX_OK;
  if (!a.offsets || !a.hmid || (need_gate_up && !a.x) || (need_down && !a.out))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  for (int e = 0; e < 2; ++e) {
    if (a.inter[e] == 0) continue;
    if ((need_gate_up && (!a.gate[e] || !a.up[e])) || (need_down && !a.down[e]))
      return fail(WX_ERR_INVALID_ARGUMENT, "%s: null weight pointer for expert %d", who, e);
  }
  const int64_t max_inter = a.inter[0] > a.inter[1] ? a.inter[0] : a.inter[1];
  if (a.rows * max_inter * 2 >= (1ll << 40)) return fail(WX_ERR_UNSUPPORTED, "%s: intermediate too large", who);
  return WX_OK;
}

// hmid_e = silu(x_e @ gate_e^T) * (x_e @ up_e^T); expert e's rows are packed with row length inter_e
int launch_gate_up(const FfnArgs& a, hipStream_t s) {
  Params p{};
  for (int e = 0; e < 2; ++e) {
    Group& g = p.g[e];
    g.a = static_cast<const __bf16*>(a.x);
    g.b0 = static_cast<const __bf16*>(a.gate[e]);
    g.b1 = static_cast<const __bf16*>(a.up[e]);
    g.c = static_cast<__bf16*>(a.hmid);
    g.m = 0; g.n = static_cast<int>(a.inter[e]); g.k = static_cast<int>(a.hidden);
    g.lda = static_cast<int>(a.hidden); g.ldb = static_cast<int>(a.hidden); g.ldc = static_cast<int>(a.inter[e]);
  }
  p.offsets = a.offsets;
  return launch_mfma<true>(p, s, "dual_gemm_kernel<swiglu>");
}

// out_e = hmid_e @ down_e^T
int launch_down(const FfnArgs& a, hipStream_t s) {
  Params p{};
  for (int e = 0; e < 2; ++e) {
    Group& g = p.g[e];
    g.a = static_cast<const __bf16*>(a.hmid);
    g.b0 = static_cast<const __bf16*>(a.down[e]);
    g.b1 = nullptr;
    g.c = static_cast<__bf16*>(a.out);
    g.m = 0; g.n = static_cast<int>(a.hidden); g.k = static_cast<int>(a.inter[e]);
    g.lda = static_cast<int>(a.inter[e]); g.ldb = static_cast<int>(a.inter[e]); g.ldc = static_cast<int>(a.hidden);
  }
  p.offsets = a.offsets;
  return launch_mfma<false>(p, s, "dual_gemm_kernel<down>");
}

}  // namespace

extern "C" int wx_dual_swiglu_gate_up(const void* x, void* hmid, const int32_t* expert_offsets, const void* gate0,
                                      const void* up0, const void* gate1, const void* up1, int64_t num_rows,
                                      int64_t hidden, int64_t inter0, int64_t inter1, wx_stream_t stream) {
  const FfnArgs a{x, {gate0, gate1}, {up0, up1}, {nullptr, nullptr}, nullptr, hmid, expert_offsets,
                  num_rows, hidden, {inter0, inter1}};
  if (int rc = check_ffn("wx_dual_swiglu_gate_up", a, true, false)) return rc;
  if (num_rows == 0) return WX_OK;
  return launch_gate_up(a, as_stream(stream));
}

extern "C" int wx_dual_down_proj(const void* hmid, void* out, const int32_t* expert_offsets, const void* down0,
                                 const void* down1, int64_t num_rows, int64_t hidden, int64_t inter0,
                                 int64_t inter1, wx_stream_t stream) {
  const FfnArgs a{nullptr, {nullptr, nullptr}, {nullptr, nullptr}, {down0, down1}, out, const_cast<void*>(hmid),
                  expert_offsets, num_rows, hidden, {inter0, inter1}};
  if (int rc = check_ffn("wx_dual_down_proj", a, false, true)) return rc;
  if (num_rows == 0) return WX_OK;
  return launch_down(a, as_stream(stream));
}

extern "C" int wx_dual_swiglu_ffn(const void* x, void* out, const int32_t* expert_offsets, const void* gate0,
                                  const void* up0, const void* down0, const void* gate1, const void* up1,
                                  const void* down1, void* hmid, int64_t num_rows, int64_t hidden, int64_t inter0,
                                  int64_t inter1, wx_stream_t stream) {
  const FfnArgs a{x, {gate0, gate1}, {up0, up1}, {down0, down1}, out, hmid, expert_offsets,
                  num_rows, hidden, {inter0, inter1}};
  if (int rc = check_ffn("wx_dual_swiglu_ffn", a, true, true)) return rc;
  if (num_rows == 0) return WX_OK;
  if (int rc = launch_gate_up(a, as_stream(stream))) return rc;
  return launch_down(a, as_stream(stream));
}
