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
#include <type_traits>

#include "common.h"

namespace wx {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 32;
constexpr int kWavesM = 2, kWavesN = 2;        // wavefront grid over the tile; one wavefront per SIMD
constexpr int kThreads = kWavesM * kWavesN * 64;
constexpr int FM = BM / kWavesM / 32;          // 32x32 accumulator blocks per wave along M (4)
constexpr int FN = BN / kWavesN / 32;          // ... and along N (4): 256 accumulator registers per lane
constexpr int kLoadRows = BM / (kWavesM * kWavesN);  // LDS rows of each operand one wave loads per K step (64)
constexpr int kLoads = kLoadRows / 16;         // 16-row load instructions per operand per wave per K step (4)
constexpr int kStages = 4;                     // ring slots per operand (the tile loop is written out for 4)
constexpr int kRowBytes = BK * 2;              // 64 bytes of K per LDS row
constexpr int kSlotBytes = BM * kRowBytes;     // 16 KiB per operand per K step
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

// s_waitcnt immediate for gfx9: vmcnt in bits [3:0] and [15:14], expcnt [6:4] (left at "no wait"), lgkmcnt [11:8]
constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | (lgkm << 8); }

struct TileCoord {
  int group, tm, tn;
};

// Linear tile id -> coordinates.  Ids are first spread so that each XCD (workgroup id mod 8) walks its own
// contiguous range of "virtual" ids; virtual ids then sweep patches of kGroupM tile rows column by column.
// Integer division runs on the vector ALU even for uniform operands, so the results are handed back through
// readfirstlane to keep everything derived from them (descriptors, branches) scalar.
__device__ __forceinline__ bool map_tile(int t, int total, const int* tiles_m, const int* tiles_n, TileCoord& tc) {
  const int per = (total + kXcds - 1) / kXcds;
  int v = (t % kXcds) * per + t / kXcds;
  if (v >= total) return false;
  int g = 0;
  const int c0 = tiles_m[0] * tiles_n[0];
  if (v >= c0) { g = 1; v -= c0; }
  const int tmn = g ? tiles_m[1] : tiles_m[0], tnn = g ? tiles_n[1] : tiles_n[0];
  const int patch = kGroupM * tnn;
  const int first_m = __builtin_amdgcn_readfirstlane(v / patch) * kGroupM;
  const int rows = tmn - first_m < kGroupM ? tmn - first_m : kGroupM;
  const int in_patch = v - (first_m / kGroupM) * patch;
  const int q = __builtin_amdgcn_readfirstlane(in_patch / rows);
  tc.group = g;
  tc.tm = first_m + (in_patch - q * rows);
  tc.tn = q;
  return true;
}

template <bool SWIGLU>
__global__ __launch_bounds__(kThreads, 1) void dual_gemm_kernel(Params p) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub; the body uses gfx950-only builtins
  // kStages ring slots per operand, each one K step (256 rows x 32 bf16).  Separate arrays let the compiler
  // see that a read of one slot never waits for a buffer load that targets another.
  __shared__ __attribute__((aligned(1024))) unsigned char s_a0[kSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_a1[kSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_a2[kSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_a3[kSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_b0[kSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_b1[kSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_b2[kSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_b3[kSlotBytes];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps descriptors and LDS bases scalar
  const int wm = wave / kWavesN, wn = wave % kWavesN;
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
  const int total = tiles_m[0] * tiles_n[0] + tiles_m[1] * tiles_n[1];  // the host bounds this below 2^31
  const int padded = (total + kXcds - 1) / kXcds * kXcds;

  // ---- per-lane constants -----------------------------------------------------------------------
  // loader: one instruction fills 16 LDS rows of 64 bytes; lane -> (row lane/4, slot lane%4).  Instruction i of
  // this wave covers rows [wave*64 + 16i, +16).  Chunk c of row r lives in slot c ^ ((r >> 2) & 3).
  const int ld_row0 = wave * kLoadRows + (lane >> 2);
  const int ld_chunk = (lane & 3) ^ ((lane >> 4) & 3);
  // fragment reads: row = base + l32, chunk kc = 2*kk + lhi
  const int sw = (l32 >> 2) & 3;
  int frag_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) frag_off[kk] = ((2 * kk + lhi) ^ sw) << 4;
  const int a_row_off = (wm * (FM * 32) + l32) * kRowBytes;
  // B fragment j of this wave starts at LDS row b_row(j): plain tiles hold 256 weight rows; SwiGLU tiles hold 128
  // gate rows then the 128 up rows of the same output columns, and fragments [0, FN/2) are gate, [FN/2, FN) up
  auto b_row = [&](int j) {
    if constexpr (SWIGLU) return (j < FN / 2 ? 0 : BN / 2) + wn * (FN / 2 * 32) + (j % (FN / 2)) * 32;
    else return wn * (FN * 32) + j * 32;
  };
  const int b_lane_off = l32 * kRowBytes;

  // ---- per-tile state ------------------------------------------------------------------------------
  struct Loader {   // where this thread's four 16-byte loads per K step come from
    const __bf16 *a_base, *b_base;
    uint32_t a_bytes, b_bytes;
    uint32_t voff_a[kLoads], voff_b[kLoads];
    int K, nk;      // nk: K steps of the tile, rounded up to a multiple of kStages (padding steps read zeros)
  };
  struct Store {    // where the finished tile goes
    __bf16* c_base;
    int rows, cols_left, ldc, nk;
  };

  auto padded_steps = [](int k) { return ((k + BK - 1) / BK + kStages - 1) / kStages * kStages; };
  auto setup_store = [&](const TileCoord& tc, Store& S) {
    const Group G = tc.group ? g1 : g0;
    const int row0 = tc.tm * BM, col0 = tc.tn * kTileN;
    S.c_base = G.c + static_cast<int64_t>(row0) * G.ldc + col0;
    S.rows = G.m - row0 < BM ? G.m - row0 : BM;
    S.cols_left = G.n - col0;
    S.ldc = G.ldc;
    S.nk = padded_steps(G.k);
  };
  auto setup_loader = [&](const TileCoord& tc, Loader& L) {
    const Group G = tc.group ? g1 : g0;
#ifdef WX_EXP_SAMETILE
    const int row0 = 0, col0 = 0;
#elif defined(WX_EXP_SAMEXCD)
    const int row0 = (blockIdx.x % 8) * BM, col0 = 0;
#else
    const int row0 = tc.tm * BM, col0 = tc.tn * kTileN;
#endif
    const int rows_a = G.m - row0 < BM ? G.m - row0 : BM;
    const int rows_b = G.n - col0 < kTileN ? G.n - col0 : kTileN;
    L.K = G.k;
    L.nk = padded_steps(G.k);
    L.a_base = G.a + static_cast<int64_t>(row0) * G.lda;
    constexpr int kHalfWaves = kWavesM * kWavesN / 2;  // SwiGLU: the first half of the waves load gate rows
    const bool up_half = SWIGLU && wave >= kHalfWaves;
    L.b_base = (up_half ? G.b1 : G.b0) + static_cast<int64_t>(col0) * G.ldb;
    L.a_bytes = static_cast<uint32_t>(rows_a) * G.lda * 2u;
    L.b_bytes = static_cast<uint32_t>(rows_b) * G.ldb * 2u;
    const int b_ld_row0 = SWIGLU ? (wave % kHalfWaves) * kLoadRows + (lane >> 2) : ld_row0;  // row inside its half
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      L.voff_a[i] = static_cast<uint32_t>(ld_row0 + 16 * i) * G.lda * 2u + ld_chunk * 16u;
      L.voff_b[i] = static_cast<uint32_t>(b_ld_row0 + 16 * i) * G.ldb * 2u + ld_chunk * 16u;
    }
  };

  // One K step of global -> LDS for this wave: rows [wave*64, +64) of the A slot and of the B slot.
  auto issue = [&](const Loader& L, int ks, unsigned char* sa, unsigned char* sb) {
    const int k0 = ks * BK;
    // advancing the base keeps the absolute end of the readable range, so rows past the matrix read as zero;
    // K chunks at or past the row end are pushed out of range per lane (this also zero-fills padding steps)
    const uint32_t adv = 2u * static_cast<uint32_t>(k0);
#ifdef WX_EXP_OOB
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(L.a_base + k0, 0u);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(L.b_base + k0, 0u);
#else
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(L.a_base + k0, L.a_bytes > adv ? L.a_bytes - adv : 0u);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(L.b_base + k0, L.b_bytes > adv ? L.b_bytes - adv : 0u);
#endif
    const bool k_tail = k0 + BK > L.K;
    const uint32_t oob = (k_tail && k0 + ld_chunk * 8 >= L.K) ? 0x80000000u : 0u;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, LDS_PTR(sa + (wave * kLoadRows + 16 * i) * kRowBytes), 16,
                                               L.voff_a[i] | oob, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, LDS_PTR(sb + (wave * kLoadRows + 16 * i) * kRowBytes), 16,
                                               L.voff_b[i] | oob, 0, 0, 0);
    }
  };

  f32x16 acc[FM][FN];
  bf16x8 fa[2][FM], fb[2][FN];  // two fragment sets: one feeds the MFMAs while the other is being read from LDS

  auto read_frags = [&](const unsigned char* sa, const unsigned char* sb, int kk, int set) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
      fa[set][i] = *reinterpret_cast<const bf16x8*>(sa + a_row_off + i * 32 * kRowBytes + frag_off[kk]);
#pragma unroll
    for (int j = 0; j < FN; ++j)
      fb[set][j] = *reinterpret_cast<const bf16x8*>(sb + b_row(j) * kRowBytes + b_lane_off + frag_off[kk]);
  };
  auto mma = [&](int set) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
  };
  // scheduling hint: the LDS reads of the next fragment set go out early among the MFMAs of this one
  auto front_load_reads = [&]() {
#pragma unroll
    for (int q = 0; q < (FM + FN) / 2; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // two LDS reads
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
    }
    __builtin_amdgcn_sched_group_barrier(0x008, FM * FN - (FM + FN) / 2, 0);
  };

  // One K step on slot (sa, sb); (sa_n, sb_n) is the next slot of the ring.  On entry fragment set 0 holds kk = 0
  // of this slot.  After the barrier every wave has finished reading this slot, so it is refilled at once with the
  // K step kStages ahead in the load stream (step `ld_ks` of tile `L`); the next slot's data was issued
  // kStages - 1 steps ago.
  auto k_step = [&](const Loader& L, int ld_ks, unsigned char* sa, unsigned char* sb, unsigned char* sa_n,
                    unsigned char* sb_n) {
    read_frags(sa, sb, 1, 1);
    mma(0);
    front_load_reads();
    // my LDS reads have returned; of my loads at most the two youngest K steps (2 * kLoads loads each) are still
    // in flight, i.e. the next slot is complete
#ifndef WX_EXP_NOWAIT
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * 2 * kLoads, 0));
#endif
#ifndef WX_EXP_NOBARRIER
    __syncthreads();
#endif
#ifndef WX_EXP_NOLOAD
    issue(L, ld_ks, sa, sb);
#endif
    __builtin_amdgcn_sched_barrier(0);  // keep the refill right behind the barrier: it has the longest way to go
    read_frags(sa_n, sb_n, 0, 0);
    mma(1);
    front_load_reads();
  };

  auto epilogue = [&](const Store& S) {
    // accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 block.
    // The lane terms are laundered through an empty asm so the per-row address arithmetic is redone here each
    // tile instead of being hoisted out of the persistent loop and held in registers across the K loop.
    int lhi_e = lhi, l32_e = l32;
    asm volatile("" : "+v"(lhi_e), "+v"(l32_e));
    const int l32 = l32_e;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wm * (FM * 32) + i * 32 + 8 * (r >> 2) + 4 * lhi_e + (r & 3);
        if (row >= S.rows) continue;
        __bf16* c_row = S.c_base + static_cast<int64_t>(row) * S.ldc;
        if constexpr (SWIGLU) {
#pragma unroll
          for (int j = 0; j < FN / 2; ++j) {
            const int col = wn * (FN / 2 * 32) + j * 32 + l32;
            if (col < S.cols_left) {
              // eager bf16 evaluation of act_fn(gate) * up (act.py:80-82): gate, up, silu(gate) and the product
              // are each rounded to bf16
              const float g = round_bf16(acc[i][j][r]);
              const float u = round_bf16(acc[i][j + FN / 2][r]);
              const float sg = round_bf16(g / (1.0f + expf(-g)));
              c_row[col] = static_cast<__bf16>(sg * u);
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            const int col = wn * (FN * 32) + j * 32 + l32;
            if (col < S.cols_left) c_row[col] = static_cast<__bf16>(acc[i][j][r]);
          }
        }
      }
    }
  };

  // ---- persistent loop -------------------------------------------------------------------------------
  // The load stream runs kStages K steps ahead of the MFMAs and crosses tile boundaries: the last kStages steps
  // of a tile refill the ring with the first kStages steps of the next tile, so the pipeline never drains and
  // the next tile's data lands while this tile's results are stored.  After the last tile the stream continues
  // with an empty descriptor (every load out of range, nothing fetched), which keeps the in-flight accounting
  // of the waits uniform.
  int next_t = blockIdx.x;
  auto next_tile = [&](TileCoord& tc) {
    bool have = false;
    for (; next_t < padded && !have; next_t += gridDim.x) have = map_tile(next_t, total, tiles_m, tiles_n, tc);
    return have;
  };
  TileCoord tc;
  bool have = next_tile(tc);
  if (!have) return;
  Loader L;
  Store S;
  setup_loader(tc, L);
  setup_store(tc, S);
  issue(L, 0, s_a0, s_b0);
  issue(L, 1, s_a1, s_b1);
  issue(L, 2, s_a2, s_b2);
  issue(L, 3, s_a3, s_b3);
  // slot 0 must be complete before its first fragments are read: three younger K steps may remain in flight
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(3 * 2 * kLoads, 15));
  __syncthreads();
  read_frags(s_a0, s_b0, 0, 0);

  while (have) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const Store done = S;
    const int nk = S.nk;
    for (int ks = 0; ks < nk; ks += kStages) {
      int ld_ks = ks + kStages;
      if (ld_ks == nk) {  // the loader moves on to the next tile (or to the empty descriptor)
        have = next_tile(tc);
        if (have) {
          setup_loader(tc, L);
          setup_store(tc, S);
        } else {
          L.a_bytes = 0;
          L.b_bytes = 0;
        }
        ld_ks = 0;
      }
      k_step(L, ld_ks + 0, s_a0, s_b0, s_a1, s_b1);
      k_step(L, ld_ks + 1, s_a1, s_b1, s_a2, s_b2);
      k_step(L, ld_ks + 2, s_a2, s_b2, s_a3, s_b3);
      k_step(L, ld_ks + 3, s_a3, s_b3, s_a0, s_b0);
    }
#ifndef WX_EXP_NOEPI
    epilogue(done);
#else
    if (acc[0][0][0] == 123.456f) epilogue(done);
#endif
  }
#endif
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
