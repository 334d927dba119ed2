// Dual asymmetric grouped GEMM and the fused dual-expert SwiGLU FFN for gfx950 (bf16 MFMA, fp32 accumulate).
//
// One persistent launch covers the tiles of BOTH experts: the grid is one workgroup per CU, the tile list is
// derived on the device from the per-expert row counts (host values, or the partition's device-side
// expert_offsets), and the tile id -> (expert, tile_m, tile_n) map keeps the 32 tiles that run concurrently on one
// XCD inside a compact patch of the output so they share operand slabs through that XCD's L2.  A skewed pair
// (thousands of VL rows next to tens of action rows, or an empty group) is just a longer or shorter tile list.
//
// Workgroup tile 256 x 256, K step 32, one workgroup per CU: eight wavefronts (two per SIMD) as 2 x 4, wave tile
// 128 x 64 = 4 x 2 MFMA 32x32x16 accumulator blocks (128 accumulator registers per lane), of which one per SIMD
// issues the global -> LDS loads; the projection that rotates heads in its epilogue runs the same tile with the
// wavefronts as 4 x 2 (wave tile 64 x 128: a wavefront holds whole heads).  Problems whose 256 x 256
// tiles would leave most CUs idle (a denoise step of a few thousand action tokens) run the same kernel with a
// 128 x 128 tile, two workgroups per CU.  A ragged last round of the fused FFN launches (tiles left over after the
// whole rounds of one tile per CU) runs in that small shape too, in a second launch, when it then fits the chip in
// one go.
// Operands are K-contiguous, so both MFMA fragments are 16-byte LDS reads.
// Global -> LDS uses buffer loads that write LDS directly (no register staging) into a ring of four K-step slots
// per operand; the load stream runs four K steps ahead of the MFMAs and crosses tile boundaries, with one
// workgroup barrier per K step.  LDS rows are 64 bytes; chunk c of row r sits in slot c ^ ((r >> 2) & 3), which
// makes the 16-byte fragment reads bank-conflict free.
//
// Operand layouts:
//   generic  (wx_dual_gemm)            A, B, C row-major; loads touch 16 rows x 64 bytes per instruction.  An
//                                      operand stored with K as its slow dimension (A as [k, m], B as [k, n]: the
//                                      backward GEMMs) is loaded as K rows of 256 columns and transposed by the LDS
//                                      reads (ds_read_b64_tr_b16), so no layout needs a transposed copy.  An
//                                      addend of C's shape can be summed in the epilogue (wx_dual_gemm_add).
//   gate/up  (wx_dual_swiglu_gate_up)  A = K-tiled activations, B = K-tiled gate and up weights (the B tile is 128
//                                      gate rows + 128 up rows of the same output columns, so gate and up of an
//                                      output element meet in one lane), C = K-tiled intermediate, SwiGLU epilogue.
//   down     (wx_dual_down_proj)       A = K-tiled intermediate, B = K-tiled down weights, C row-major; with a row
//                                      id list the rows go straight to their token positions (the unpermute), and
//                                      a residual matrix can be added there on the way (the layer's closing add).
//   qkv+rope (wx_qkv_rope_proj)        A, B, C row-major like the generic mode, one group; bias and the rotary
//                                      embedding of the q and k heads are applied to the accumulators.
// With K-tiled operands every load instruction moves one contiguous KiB (tiled_layout.h).
// Results leave through a per-wave LDS staging area so that global stores are full 16-byte lanes on contiguous
// runs (whole 1 KiB blocks for the tiled intermediate, 256-byte row segments for row-major outputs).
#include <type_traits>

#include "common.h"
#include "tiled_layout.h"

namespace wx {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BK = 32;
constexpr int kStages = 4;                     // ring slots per operand
constexpr int kRowBytes = BK * 2;              // 64 bytes of K per LDS row

// Workgroup tile shapes.  Everything else (wave tile, loads per step, LDS footprint, resident workgroups per CU)
// follows from the two numbers.
// LW_: how many of the wavefronts (the first LW_) issue the global -> LDS loads; 0 = all of them.
template <int BM_, int BN_, int WM_, int WN_, int LW_ = 0>
struct TileShape {
  static constexpr int BM = BM_, BN = BN_;
  static constexpr int kWavesM = WM_, kWavesN = WN_;  // wavefront grid over the tile
  static constexpr int kWaves = kWavesM * kWavesN;
  static constexpr int kLoadWaves = LW_ > 0 ? LW_ : kWaves;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int FM = BM / kWavesM / 32;        // 32x32 accumulator blocks per wave along M
  static constexpr int FN = BN / kWavesN / 32;        // ... and along N
  static constexpr int kLoadRowsA = BM / kLoadWaves;  // LDS rows of A one loading wave loads per K step
  static constexpr int kLoadRowsB = BN / kLoadWaves;  // ... and of B
  static constexpr int kLoadsA = kLoadRowsA / 16;     // 16-row load instructions per wave per K step: A
  static constexpr int kLoadsB = kLoadRowsB / 16;     // ... and B
  static constexpr int kSlotBytesA = BM * kRowBytes;  // bytes of A per K step
  static constexpr int kSlotBytesB = BN * kRowBytes;
  static constexpr int kStageBytes = FN >= 4 ? (kWaves > 4 || BM <= 128 ? 4096 : 8192) : 2048;  // per-wave staging for the epilogue
  static constexpr int kLdsBytes = kStages * (kSlotBytesA + kSlotBytesB) + kWaves * kStageBytes;
  static constexpr int kWgPerCu = kLdsBytes <= 80 * 1024 && FM * FN * 16 <= 128 ? 2 : 1;
  static_assert(kLdsBytes <= 160 * 1024, "LDS budget");
  static_assert(FM >= 1 && FN >= 2 && FN % 2 == 0 && kLoadsA >= 1 && kLoadsB >= 1 && kLoadsB <= kLoadsA, "tile shape");
};
// four wavefronts (one per SIMD) as 2 x 2: wave tile 128 x 128, 256 accumulator registers per lane
using BigTile = TileShape<256, 256, 2, 2>;
// eight wavefronts (two per SIMD) as 2 x 4: wave tile 128 x 64, 128 accumulator registers per lane, and only the
// first four (one per SIMD) issue the global -> LDS loads.  A wavefront that issues a load stalls while the CU's load
// path takes the instruction in; here its partner on the same SIMD issues no loads and keeps the MFMA pipe fed
// meanwhile.  Against BigTile, on the config 3 shapes: gate/up 4-7 % faster, down 3 %, the row-major op 2-6 %.
// (With all eight loading on one schedule, both partners stall together: that form was 2 % ahead of BigTile on
// gate/up and behind it elsewhere.)
using BigTile8 = TileShape<256, 256, 2, 4, 4>;
// The small tile, for problems with too few large tiles to fill the chip: two workgroups per CU, each eight
// wavefronts as 4 x 2 (wave tile 32 x 64), four of them loading, like the large tile.  (Four wavefronts of 64 x 64
// measure 6 % slower on a denoise step; timestamps inside that kernel put 254 ns on a K step whose 8 MFMAs per
// wavefront need 110, and 169 ns with the loads taken out.)
using SmallTile = TileShape<128, 128, 4, 2, 4>;
// the same eight wavefronts as 4 x 2: wave tile 64 x 128, for the epilogue that needs a wavefront to hold whole
// 128-column heads (the rotation partner of a channel is 64 columns away)
using BigTile8Q = TileShape<256, 256, 4, 2, 4>;
// The large tile of a launch.
template <int MODE>
using BigTileFor = std::conditional_t<MODE == 3 || MODE == 4 /* kQkvRope, kQkvRopeFull */, BigTile8Q, BigTile8>;
// the shape that runs the ragged last round of a launch (see tail_split_point): BigTile cut in four.  (Cut in two,
// 256 x 128 with one workgroup per CU, measures the same.)
using TailTile = SmallTile;
// ... and for the projection that rotates heads: four wavefronts as 4 x 1, wave tile 32 x 128, so that a wavefront
// still holds whole heads of 128 channels (all four load)
using TailTileQ = TileShape<128, 128, 4, 1>;
template <int MODE>
using TailTileFor = std::conditional_t<MODE == 3 || MODE == 4 /* kQkvRope, kQkvRopeFull */, TailTileQ, TailTile>;

constexpr int kXcds = 8;
constexpr int kGroupM = 8;                     // tile rows per patch in the tile order

// kQkvRopeFull: kQkvRope reading a rotary table with one entry per channel (an instantiation of its own: both table
// forms in one kernel cost the K loop registers)
enum Mode { kGeneric = 0, kGateUp = 1, kDown = 2, kQkvRope = 3, kQkvRopeFull = 4 };

struct Group {
  const __bf16* a;   // generic: [m, k] row-major (lda).  tiled: base of the K-tiled matrix
  const __bf16* b0;  // generic: [n, k] row-major (ldb).  tiled: K-tiled weights (gate for kGateUp)
  const __bf16* b1;  // kGateUp: K-tiled up weights
  __bf16* c;         // row-major [m, n] (ldc), or base of the K-tiled intermediate (kGateUp)
  int m, n, k;
  int lda, ldb, ldc;  // row-major: leading dimension in elements.  tiled: number of 16-row blocks of the matrix
  int a_row0;         // tiled A: first row of this group inside the tiled matrix (a multiple of 256)
  const __bf16* add;  // generic: optional [m, n] row-major (ldc) matrix added to the product (may be c itself)
};

struct Params {
  Group g[2];
  const int32_t* offsets;  // device int32[3]: rows of expert e are [offsets[e], offsets[e+1]); null for kGeneric
  // Tile-shape choice made on the device, for launches where the host cannot tell (the split of the rows between
  // the experts lives in `offsets`): both tile shapes are launched and each kernel returns at once unless the
  // number of 256 x 256 tiles is on its side of `gate_tiles`.  0 = always run, 1 = run if at most gate_tiles,
  // 2 = run if more.
  int gate, gate_tiles;
  // Tail split (see tail_split_point): 0 = off; 1 = this launch does the whole rounds of 256 x 256 tiles and leaves
  // the ragged last round to a second launch; 2 = this is that second launch, with 128 x 128 tiles.
  // split_cus = workgroups of the first launch (one per CU).
  int split, split_cus;
  // kDown only: when set (the partition's sorted_row_id), row r of the sorted result is stored to row scatter[r] of
  // the output instead of row r -- the unpermute folded into the store.
  const int32_t* scatter;
  // kDown with scatter only: when set, a [tokens, n] matrix laid out like the output whose rows are added to the
  // result before the store (out[t] = residual[t] + y[t], each term bf16, one rounding) -- the decoder layer's
  // closing residual add.  May be the output itself.
  const __bf16* residual;
  // kQkvRope only (group 0 is the projection, row-major operands): bias[n] (may be null), the packed rotary table
  // [m, rope_width] (bf16 cos | bf16 sin << 16 per token and channel: rope_width 64 when channels d and d + 64 share
  // an entry, 128 when every channel has its own) and the number of leading output columns that are rotated (whole
  // heads of 128: the q and k heads; the v heads behind them only take the bias).
  const __bf16* bias;
  const uint32_t* rope_table;
  int rope_cols, rope_width;
  // kGateUp only (training): when set, the two projections themselves (rounded to bf16, before the SwiGLU) are
  // stored as well, K-tiled with the geometry of the intermediate, so that a backward pass need not recompute them.
  __bf16* keep_gate;
  __bf16* keep_up;
};

#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define LDS_TR_PTR(p) ((__attribute__((address_space(3))) bf16x4*)(p))

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
__device__ __forceinline__ void tile_coords(int v, const int* tiles_m, const int* tiles_n, TileCoord& tc) {
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
}
// The share of `n` tiles that XCD `x` walks when they are dealt out as evenly as possible, the XCDs taking their
// places in the dealing order from `first` on (the first n % 8 places get one tile more): how many, and the index of
// the first one (every XCD's share is a contiguous range).
__device__ __forceinline__ void xcd_share(int n, int x, int first, int& count, int& start) {
  const int q = n / kXcds, r = n % kXcds;
  const int pos = (x - first + kXcds) % kXcds;
  count = q + (pos < r ? 1 : 0);
  start = pos * q + (pos < r ? pos : r);
}
// Workgroup slot t (XCD t % 8, place t / 8 among that XCD's workgroups and rounds) -> tile.  Each expert's tiles
// are dealt to the XCDs separately, expert 1's starting at the XCD where expert 0's remainder ended, so every XCD
// walks its share of expert 0 and then its share of expert 1, at most ceil(total / 8) tiles in all.  With one list
// cut into eight ranges instead, a short second expert would sit at the end of the last XCD's range alone: cheap
// tiles (the action expert's down projection, a tenth of the contraction) then replace expensive ones on one XCD
// only, and the other seven run a longer list.
__device__ __forceinline__ bool map_tile(int t, int total, const int* tiles_m, const int* tiles_n, TileCoord& tc) {
  const int all0 = tiles_m[0] * tiles_n[0];
  const int n0 = all0 < total ? all0 : total, n1 = total - n0;  // (a first launch of a tail split stops at `total`)
  const int x = t % kXcds, j = t / kXcds;
  int count, start;
  xcd_share(n0, x, 0, count, start);
  int v = start + j;
  if (j >= count) {
    const int j1 = j - count;
    xcd_share(n1, x, n0 % kXcds, count, start);
    if (j1 >= count) return false;
    v = n0 + start + j1;
  }
  tile_coords(v, tiles_m, tiles_n, tc);
  return true;
}

// The ragged last round.  `total` 256 x 256 tiles on `cus` workgroups take ceil(total / cus) rounds however few
// tiles the last round holds.  When the tiles left over after the whole rounds (in virtual-id order: the last tile
// rows of expert 0, then expert 1) fit the chip as 128 x 128 tiles in one go -- four per large tile, two workgroups
// per CU -- the first launch stops at the whole rounds and a second launch runs the rest in the small shape.
// Tiles of an expert whose contraction is at most half as long as the other's are cheap enough to ride along
// as a second helping and are not counted.  Returns the number of tiles of the first launch
// (== total: no split).  Evaluated identically by the host (when it knows the row counts) and by both launches.
__host__ __device__ inline int tail_split_point(int tiles0, int tiles1, int k0, int k1, int cus) {
  const int total = tiles0 + tiles1;
  if (cus <= 0 || total <= cus) return total;
  const int full = total / cus * cus, tail = total - full;
  if (tail == 0) return total;
  const int tail1 = tail < tiles1 ? tail : tiles1, tail0 = tail - tail1;
  const int counted = (tiles1 > 0 && tiles0 > 0 && 2ll * k1 <= k0) ? tail0 : tail;
  return 2 * counted <= cus ? full : total;
}

// The tile count that decides between the two tile shapes.  The small shape pays when the large tiles would leave
// half of the CUs idle.  Tiles of an expert whose contraction is at most half as long as the other's do not count:
// in the small shape they ride along as a cheap second helping of the first workgroups (4096 VL rows next to a
// handful of action rows in the down launch: 128 tiles of K = 11008 and 8 of K = 1024 are one round of small tiles
// plus a tenth, not 136 large tiles on 256 CUs).  Evaluated identically by the host and by both launches.
__host__ __device__ inline long long shape_deciding_tiles(long long tiles0, long long tiles1, int k0, int k1) {
  if (tiles0 > 0 && tiles1 > 0) {
    if (2ll * k1 <= k0) return tiles0;
    if (2ll * k0 <= k1) return tiles1;
  }
  return tiles0 + tiles1;
}

// Workgroup barrier without the fences of __syncthreads().  Those fences make the compiler wait for EVERY
// outstanding LDS-direct load (vmcnt(0)) at the barrier, which drains the prefetch ring on each K step; the waits
// the data flow needs (own LDS reads returned, own loads of the next slot landed) are written out before each call.
// The empty asm statements keep the compiler from moving memory accesses across the barrier.
__device__ __forceinline__ void barrier_no_fence() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const bf16x2 v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};  // one packed convert
  return __builtin_bit_cast(uint32_t, v);
}

// One LDS array per (size, alignment, index).
template <int BYTES, int ALIGN, int ID>
__device__ __forceinline__ unsigned char* lds_array() {
  __shared__ __attribute__((aligned(ALIGN))) unsigned char s[BYTES];
  return s;
}

// The fused FFN launch: gate/up tiles (producers) and down tiles (consumers) in one grid.  A down tile of row block
// rb reads the intermediate rows that the gate/up tiles of the same row block write, so it waits until `ready[rb]`
// has reached the number of those tiles.  An XCD places its share of a launch's workgroups in index order and the
// producers come first, so on every XCD the producers have their places before a consumer gets one, and producers
// never wait: a launch alone on the chip always makes progress.  So do two of them in flight together on their own
// workspaces (an XCD has 64 places for workgroups of this size, a launch at most 32 consumers per XCD, and a
// launch's consumers hold no place on an XCD where its producers still wait for one: waiting workgroups cannot
// fill an XCD).  The wait is bounded all the same (kFusedWaitTicks of the 100 MHz clock; then `*error` is set and
// the tile goes ahead on whatever is there), which is what three or more concurrent launches would fall back on.  The last consumer past the wait of a row block clears the row block's counters, so a launch
// leaves the workspace as it found it: all zero.
// The producers can read their A operand from the token rows themselves (AROWS below: `x` through `gather`), which
// makes the permute into the K-tiled activation matrix part of the launch.
constexpr int kFusedMaxRowBlocks = 256;   // 128-row blocks per expert
constexpr long long kFusedWaitTicks = 500000000ll;  // 5 s
constexpr int kFusedCounterStride = 64;   // ints between two counters: 256 bytes, so that the polls of different row
                                          // blocks (and the increments) spread over the memory channels
constexpr int kFusedCounters = 2 * kFusedMaxRowBlocks * kFusedCounterStride;  // ints of one counter array
struct FusedSync {
  int* ready;     // [2 * kFusedMaxRowBlocks] x stride: gate/up tiles finished, by expert and row block
  int* passed;    // ... down tiles past their wait
  int* error;     // set to 1 when a wait ran into its bound
  int need[2];    // gate/up tiles per row block of expert e
  const __bf16* warm_b[2][2];  // the producers' weights (gate, up of expert e), K-tiled; null: nothing to warm
  int warm_ldb[2];             // their row blocks per column block
  int warm_k;                  // their contraction length
  int consumers;  // down tiles per row block
  // AROWS: the activations in token order, [tokens, hidden] bf16 row-major, and the partition's sorted_row_id
  // (sorted position -> token)
  const __bf16* x;
  const int32_t* gather;
};

// KA / KB (generic mode only): the operand is stored with K as its slow dimension -- A as [k, m], B as [k, n] --
// and is transposed on the way from LDS to the MFMA registers.
//
// The kernel's body is a function of its own so that one launch can run two of them side by side (the fused FFN
// launch below: some workgroups run the gate/up form, the others the down form).  `wg` of `n_wg` is the workgroup's
// place among those that share this body's tile list (blockIdx.x of gridDim.x in a plain launch).
// ROLE: 0 = a plain launch; 1 / 2 = producer / consumer of a fused launch (see FusedSync).  AROWS (gate/up form of a fused launch): the A operand is read from the token rows themselves,
// fs.x through fs.gather, instead of from a K-tiled copy of them.
template <int MODE, typename TS, bool KA, bool KB, int ROLE, bool AROWS = false>
__device__ __forceinline__ void dual_gemm_body(const Params& p, const int wg, const int n_wg, const FusedSync& fs) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub; the body uses gfx950-only builtins
  constexpr int BM = TS::BM, BN = TS::BN, FM = TS::FM, FN = TS::FN;
  constexpr int kWavesN = TS::kWavesN, kWaves = TS::kWaves;
  constexpr int kLoadRowsA = TS::kLoadRowsA, kLoadRowsB = TS::kLoadRowsB, kLoadsA = TS::kLoadsA, kLoadsB = TS::kLoadsB;
  constexpr int kLoadsPerStep = kLoadsA + kLoadsB;
  constexpr int kSlotBytesA = TS::kSlotBytesA, kSlotBytesB = TS::kSlotBytesB, kStageBytes = TS::kStageBytes;
  constexpr bool SWIGLU = MODE == kGateUp;
  constexpr bool TILED_IN = MODE == kGateUp || MODE == kDown;   // A and B are K-tiled
  constexpr bool TILED_OUT = MODE == kGateUp;   // C is K-tiled
  static_assert(MODE == kGeneric || (!KA && !KB), "K-major operands exist in the generic mode only");
  // kStages ring slots per operand, each one K step (256 rows x 32 bf16).  Separate arrays let the compiler
  // see that a read of one slot never waits for a buffer load that targets another.
  // Row-major operands with K contiguous (the NT layout of the generic mode): the ring's slots live in PAIRS.  A load instruction then fetches 8 rows x 128 bytes -- the K chunks of two consecutive K steps,
  // i.e. whole cache lines -- where one slot's worth would be 16 rows x 64 bytes (sixteen half lines, which hold the
  // loading wavefront's issue slot about twice as long).  A pair is one array of 1 KiB blocks, block = 8 rows x
  // [512 bytes of the even step | 512 bytes of the odd step], so the instruction's 64 lanes land on consecutive LDS
  // addresses; inside a step's half, rows are 64 bytes with the same chunk swizzle as everywhere else.
  // (The projection that rotates heads reads row-major operands too and keeps the slot-by-slot ring: with pairs its
  // launches measured 3 % slower inside a forward pass.)
  constexpr bool kPair = MODE == kGeneric && !KA && !KB;
  // NN (a row-major A beside a K-major B: dX, dHm, the op's default layout): A alone lives in pairs, B keeps its slots
  constexpr bool kPairAOnly = MODE == kGeneric && !KA && KB;
  constexpr bool kPA = kPair || kPairAOnly, kPB = kPair;
  constexpr int kRingA = kPA ? 16 : kSlotBytesA, kRingB = kPB ? 16 : kSlotBytesB;  // the form not in use shrinks
  constexpr int kPairA = kPA ? 2 * kSlotBytesA : 16, kPairB = kPB ? 2 * kSlotBytesB : 16;
  constexpr int kRingAlignA = kPA ? 16 : 1024, kPairAlignA = kPA ? 1024 : 16;
  constexpr int kRingAlignB = kPB ? 16 : 1024, kPairAlignB = kPB ? 1024 : 16;
  // (one LDS object per (size, alignment, index): the two bodies of a fused launch name the same objects, so the
  // launch needs the LDS of one of them)
  unsigned char* const s_a0 = lds_array<kRingA, kRingAlignA, 0>();
  unsigned char* const s_a1 = lds_array<kRingA, kRingAlignA, 1>();
  unsigned char* const s_a2 = lds_array<kRingA, kRingAlignA, 2>();
  unsigned char* const s_b0 = lds_array<kRingB, kRingAlignB, 3>();
  unsigned char* const s_b1 = lds_array<kRingB, kRingAlignB, 4>();
  unsigned char* const s_b2 = lds_array<kRingB, kRingAlignB, 5>();
  unsigned char* const s_a3 = lds_array<kRingA, kRingAlignA, 6>();
  unsigned char* const s_b3 = lds_array<kRingB, kRingAlignB, 7>();
  unsigned char* const s_pa0 = lds_array<kPairA, kPairAlignA, 8>();  // slots 0 and 1 of A
  unsigned char* const s_pa1 = lds_array<kPairA, kPairAlignA, 9>();  // slots 2 and 3
  unsigned char* const s_pb0 = lds_array<kPairB, kPairAlignB, 10>();
  unsigned char* const s_pb1 = lds_array<kPairB, kPairAlignB, 11>();
  unsigned char* const s_out = lds_array<kWaves * kStageBytes, 1024, 12>();
  // ring slot s of each operand (s is a constant after unrolling)
  static_assert(kStages == 4, "ring slots are declared one by one");
  auto slot_a = [&](int s) -> unsigned char* {
    if constexpr (kPA) return (s < 2 ? s_pa0 : s_pa1) + (s & 1) * 512;
    else return s == 0 ? s_a0 : (s == 1 ? s_a1 : (s == 2 ? s_a2 : s_a3));
  };
  auto slot_b = [&](int s) -> unsigned char* {
    if constexpr (kPB) return (s < 2 ? s_pb0 : s_pb1) + (s & 1) * 512;
    else return s == 0 ? s_b0 : (s == 1 ? s_b1 : (s == 2 ? s_b2 : s_b3));
  };

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps descriptors and LDS bases scalar
  const int wm = wave / kWavesN, wn = wave % kWavesN;
  const int l32 = lane & 31, lhi = lane >> 5;
  // With more wavefronts than SIMDs only the first kLoadWaves (one per SIMD) issue the global -> LDS loads.  A
  // wavefront that issues a load is held while the CU's load path takes the instruction in; its partner on the same
  // SIMD, which issues none, keeps the MFMA pipe fed meanwhile.  When both partners load on the same schedule they
  // stall together and the pipe idles.
  constexpr int kLoadWaves = TS::kLoadWaves;
  constexpr bool ASYM = kLoadWaves != kWaves;
  const bool loads = !ASYM || wave < kLoadWaves;

  // ---- problem table (uniform) ------------------------------------------------------------------
  // (kept as two named structs, selected per tile, so everything stays in scalar registers)
  Group g0 = p.g[0], g1 = p.g[1];
  int sorted_first[2] = {0, 0};  // tiled modes: sorted position of each expert's first row
  int sorted_total = 0;          // ... and the number of sorted rows
  if constexpr (TILED_IN) {
    const int o0 = p.offsets[0], o1 = p.offsets[1], o2 = p.offsets[2];
    g0.m = o1 - o0;
    g1.m = o2 - o1;
    const int pad0 = static_cast<int>(round_up_256(g0.m)), pad1 = static_cast<int>(round_up_256(g1.m));
    if constexpr (MODE == kGateUp) {
      // A: one tiled activation matrix, expert 1 starts at the next multiple of 256 rows.
      // C: per-expert tiled intermediates, packed one after the other
      g0.a_row0 = 0;
      g1.a_row0 = pad0;
      g0.ldc = pad0 / kBlkRows;
      g1.ldc = pad1 / kBlkRows;
      g1.c = g0.c + static_cast<int64_t>(pad0) * g0.n;
    } else {
      // A: per-expert tiled intermediates;  C: row-major, expert e's rows start at offsets[e]
      g0.a_row0 = 0;
      g1.a_row0 = 0;
      g0.lda = pad0 / kBlkRows;
      g1.lda = pad1 / kBlkRows;
      g1.a = g0.a + static_cast<int64_t>(pad0) * g0.k;
      if (p.scatter == nullptr) {
        g0.c += static_cast<int64_t>(o0) * g0.ldc;
        g1.c += static_cast<int64_t>(o1) * g1.ldc;
      }
    }
    sorted_first[0] = o0;
    sorted_first[1] = o1;
    sorted_total = o2;
  }
  constexpr int kTileN = SWIGLU ? BN / 2 : BN;  // output columns per tile
  int tiles_m[2], tiles_n[2];
  tiles_m[0] = (g0.m + BM - 1) / BM;
  tiles_n[0] = (g0.n + kTileN - 1) / kTileN;
  if (g0.m <= 0 || g0.n <= 0) tiles_m[0] = tiles_n[0] = 0;
  tiles_m[1] = (g1.m + BM - 1) / BM;
  tiles_n[1] = (g1.n + kTileN - 1) / kTileN;
  if (g1.m <= 0 || g1.n <= 0) tiles_m[1] = tiles_n[1] = 0;
  if (p.gate != 0) {
    constexpr int kBigN = SWIGLU ? BigTile::BN / 2 : BigTile::BN;
    auto big = [](int m, int n) { return (m <= 0 || n <= 0) ? 0 : ((m + BigTile::BM - 1) / BigTile::BM) * ((n + kBigN - 1) / kBigN); };
    const bool few = shape_deciding_tiles(big(g0.m, g0.n), big(g1.m, g1.n), g0.k, g1.k) <= p.gate_tiles;
    if (few != (p.gate == 1)) return;  // uniform: the other tile shape's launch does this problem
  }
  int total = tiles_m[0] * tiles_n[0] + tiles_m[1] * tiles_n[1];  // the host bounds this below 2^31
  // tail split: the first launch (256 x 256 tiles) stops at `split_at`; the second (this shape: 128 x 128)
  // takes virtual tiles [split_at, all) of the 256 x 256 tiling, kSubM x kSubN pieces each
  constexpr bool kIsTail = std::is_same_v<TS, TailTileFor<MODE>>, kIsBig = std::is_same_v<TS, BigTileFor<MODE>>;
  constexpr int kSubM = BigTile::BM / BM, kSubN = BigTile::BN / BN;
  int big_m[2], big_n[2], split_at = 0, pieces = 0;
  if ((kIsBig && p.split == 1) || (kIsTail && p.split == 2)) {
    constexpr int kBigN = SWIGLU ? BigTile::BN / 2 : BigTile::BN;
    big_m[0] = (g0.m + BigTile::BM - 1) / BigTile::BM;
    big_n[0] = (g0.n + kBigN - 1) / kBigN;
    if (g0.m <= 0 || g0.n <= 0) big_m[0] = big_n[0] = 0;
    big_m[1] = (g1.m + BigTile::BM - 1) / BigTile::BM;
    big_n[1] = (g1.n + kBigN - 1) / kBigN;
    if (g1.m <= 0 || g1.n <= 0) big_m[1] = big_n[1] = 0;
    const int all = big_m[0] * big_n[0] + big_m[1] * big_n[1];
    split_at = tail_split_point(big_m[0] * big_n[0], big_m[1] * big_n[1], g0.k, g1.k, p.split_cus);
    if constexpr (kIsBig) {
      total = split_at;  // a multiple of 8 when smaller than `all`
    } else {
      if (split_at == all) return;  // no split: the first launch did everything
      pieces = kSubM * kSubN * (all - split_at);
    }
  }
  const int padded = (total + kXcds - 1) / kXcds * kXcds;

  // ---- per-lane constants -----------------------------------------------------------------------
  // row-major loader: one instruction fills 16 LDS rows of 64 bytes; lane -> (row lane/4, slot lane%4).
  // Instruction i of this wave covers rows [wave*64 + 16i, +16) of A.  Chunk c of row r lives in slot c ^ ((r >> 2) & 3).
  const int ld_row0 = wave * kLoadRowsA + (lane >> 2);
  const int ld_chunk = (lane & 3) ^ ((lane >> 4) & 3);
  // fragment reads: row = base + l32, chunk kc = 2*kk + lhi
  const int sw = (l32 >> 2) & 3;
  int frag_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) frag_off[kk] = ((2 * kk + lhi) ^ sw) << 4;
  const int a_row_off = (wm * (FM * 32) + l32) * kRowBytes;
  // paired slots: row r of a step's half sits at block r / 8 (1 KiB each), row r % 8 inside it
  const int pair_lane_off = ((l32 >> 3) << 10) + ((l32 & 7) << 6);
  const int a_pair_off = wm * (FM * 32) * 128 + pair_lane_off;
  // paired loader: lane -> (row lane / 4 % 8 of the instruction's 8 rows, step half lane / 32, slot lane % 4)
  constexpr int kPairLoadsA = kLoadRowsA / 8, kPairLoadsB = kLoadRowsB / 8;
  const int pl_row = (lane >> 2) & 7, pl_half = lane >> 5, pl_slot = lane & 3;
  // K chunk (of the 8 in a 128-byte line) this lane fetches in instruction i: the instruction's rows are 8 i + pl_row
  // past a multiple of 32, and the slot holds chunk slot ^ ((row >> 2) & 3) of its step -- one value for even i, one
  // for odd i, so a lane's byte offsets are two bases plus i times the (uniform) pitch of 8 rows
  const int pair_chunk_even = 4 * pl_half + (pl_slot ^ ((pl_row >> 2) & 3));
  const int pair_chunk_odd = 4 * pl_half + (pl_slot ^ (((pl_row >> 2) + 2) & 3));
  auto pair_chunk = [&](int i) { return (i & 1) ? pair_chunk_odd : pair_chunk_even; };
  // B fragment j of this wave starts at LDS row b_row(j): plain tiles hold 256 weight rows; SwiGLU tiles hold 128
  // gate rows then the 128 up rows of the same output columns, and fragments [0, FN/2) are gate, [FN/2, FN) up
  auto b_row = [&](int j) {
    if constexpr (SWIGLU) return (j < FN / 2 ? 0 : BN / 2) + wn * (FN / 2 * 32) + (j % (FN / 2)) * 32;
    else return wn * (FN * 32) + j * 32;
  };
  const int b_lane_off = l32 * kRowBytes;
  // K-major operand (KA / KB): a slot holds BK rows of K, each a run of BM (BN) columns, as whole 16-byte chunks;
  // the 64-byte segment s of row k sits at segment position s ^ (k & 3), so that the four rows one transposing
  // read touches fall into different banks.  ds_read_b64_tr_b16 works on groups of 16 lanes: lane j of a group
  // supplies the address of 4 consecutive columns of row (j >> 2), and receives column j of the 4 rows.  A group
  // covers 16 columns; the two groups of a half-wave cover a 32-column block, the half-waves rows k and k + 8.
  const int tr_j = lane & 15, tr_grp = (lane >> 4) & 1;
  const int tr_in = (2 * tr_grp + ((tr_j >> 1) & 1)) * 16 + 8 * (tr_j & 1);  // bytes inside the 64-byte segment
  auto tr_lane_base = [&](int row_bytes, int first_block) {  // first_block: this wave's first 32-column block
    return (8 * lhi + (tr_j >> 2)) * row_bytes + ((first_block ^ (tr_j >> 2)) << 6) + tr_in;
  };
  const int tr_base_a = KA ? tr_lane_base(BM * 2, wm * FM) : 0;
  const int tr_base_b = KB ? tr_lane_base(BN * 2, wn * FN) : 0;

  // ---- per-tile state ------------------------------------------------------------------------------
  struct Loader {   // where this wave's kLoadsA + kLoadsB loads per K step come from
    const __bf16 *a_base, *b_base;
    uint32_t a_bytes, b_bytes;        // readable bytes from the base (row-major) / from the current block (tiled)
    uint32_t voff_a[kPA ? 2 : kLoadsA], voff_b[kPB ? 2 : kLoadsB];  // paired slots: [even i, odd i] of instruction 0
    uint32_t pitch8_a, pitch8_b;      // paired slots: bytes between the rows of consecutive load instructions
    int64_t a_step, b_step;           // tiled: bytes between consecutive K steps
    // tiled: the load stream walks a tile's K steps in order, so the step's base and the bytes readable from it are
    // kept as running values (one add and one saturating subtract per step) instead of products with the step index
    const char *a_cur, *b_cur;
    uint32_t a_left, b_left, a_dec, b_dec;
    int K, nk;      // nk: K steps of the tile, rounded up to a multiple of kStages (padding steps read zeros)
  };
  struct Store {    // where the finished tile goes
    __bf16* c_base;
    const int32_t* row_id;  // kDown with scatter: output row of each of the tile's rows (c_base is then row 0)
    const __bf16* res;      // kDown with scatter and a residual: the residual's column col0 of row 0; generic with
                            // an addend: its element under c_base; else null
    int rows, cols_left, ldc, nk;
    int row0, col0;         // first row / column of the tile inside its group's output
    int row_block;          // fused launch: index of the tile's (expert, row block) counters
  };

  // K steps of a tile rounded up to whole ring rounds (padding steps read zeros).  The host never launches this
  // kernel with k == 0 and a non-empty output: the tile loop below advances only from inside the K loop.
  auto padded_steps = [](int k) { return ((k + BK - 1) / BK + kStages - 1) / kStages * kStages; };
  auto setup_store = [&](const TileCoord& tc, Store& S) {
    const Group G = tc.group ? g1 : g0;
    const int row0 = tc.tm * BM, col0 = tc.tn * kTileN;
    if constexpr (TILED_OUT) {
      // block (row block, column block) of the tiled intermediate: [column block][row block], 1 KiB each
      S.c_base = G.c + ((static_cast<int64_t>(col0 / kBlkCols) * G.ldc + row0 / kBlkRows) << 9);
    } else {
      S.c_base = G.c + static_cast<int64_t>(row0) * G.ldc + col0;
    }
    S.row_id = nullptr;
    S.res = nullptr;
    if constexpr (MODE == kDown) {
      if (p.scatter != nullptr) {
        S.c_base = G.c + col0;
        S.row_id = p.scatter + sorted_first[tc.group] + row0;
        if (p.residual != nullptr) S.res = p.residual + col0;
      }
    }
    if constexpr (MODE == kGeneric) {
      if (G.add != nullptr) S.res = G.add + static_cast<int64_t>(row0) * G.ldc + col0;
    }
    S.rows = G.m - row0 < BM ? G.m - row0 : BM;
    S.cols_left = G.n - col0;
    S.row0 = row0;
    S.col0 = col0;
    S.row_block = tc.group * kFusedMaxRowBlocks + tc.tm;
    S.ldc = G.ldc;
    S.nk = padded_steps(G.k);
  };
  auto setup_loader = [&](const TileCoord& tc, Loader& L) {
    const Group G = tc.group ? g1 : g0;
    const int row0 = tc.tm * BM, col0 = tc.tn * kTileN;
    L.K = G.k;
    L.nk = padded_steps(G.k);
    constexpr int kHalfWaves = kLoadWaves / 2;  // SwiGLU: the first half of the loading waves load gate rows, the rest up rows
    const bool up_half = SWIGLU && wave >= kHalfWaves;
    const __bf16* b_src = up_half ? G.b1 : G.b0;
    const int b_wave = SWIGLU ? wave % kHalfWaves : wave;
    if constexpr (TILED_IN) {
      // this wave's row blocks of the A tile and of the B tile at K step 0; a K step later they sit one column
      // block further, i.e. (row blocks of the matrix) KiB ahead
      const int64_t b_blk = col0 / kBlkRows + b_wave * kLoadsB;
      L.b_base = b_src + (b_blk << 9);
      L.b_step = static_cast<int64_t>(G.ldb) << 10;
      const int64_t b_left = (static_cast<int64_t>(G.k / kBlkCols) * G.ldb - b_blk) << 10;
      L.b_bytes = static_cast<uint32_t>(b_left < 0 ? 0 : (b_left > 0x7fffff00ll ? 0x7fffff00ll : b_left));
      L.b_cur = reinterpret_cast<const char*>(L.b_base);
      L.b_left = L.b_bytes;
      L.b_dec = static_cast<uint32_t>(L.b_step > 0x7fffff00ll ? 0x7fffff00ll : L.b_step);
#pragma unroll
      for (int i = 0; i < kLoadsB; ++i) L.voff_b[i] = static_cast<uint32_t>(i * kBlkBytes + lane * 16);
      if constexpr (AROWS) {
        // A from the token rows: sorted row r of the tile is row gather[...] of the row-major activations; a load
        // instruction fetches 64 bytes of 16 such rows (lane -> row lane / 4, and the chunk that belongs in LDS slot
        // lane % 4), rows past the expert's last row read as zero.  The host keeps the matrix below 2 GiB.
        const int rows_a = G.m - row0 < BM ? G.m - row0 : BM;
        L.a_base = fs.x;
        L.a_bytes = static_cast<uint32_t>(sorted_total) * static_cast<uint32_t>(G.k) * 2u;
        L.a_step = 0;
        L.a_cur = nullptr;
        L.a_left = L.a_dec = 0;
#pragma unroll
        for (int i = 0; i < kLoadsA; ++i) {
          const int r = ld_row0 + 16 * i;
          uint32_t v = 0x80000000u;
          if (r < rows_a)
            v = static_cast<uint32_t>(fs.gather[sorted_first[tc.group] + row0 + r]) * static_cast<uint32_t>(G.k) * 2u + ld_chunk * 16u;
          L.voff_a[i] = v;
        }
      } else {
        const int64_t a_blk = (G.a_row0 + row0) / kBlkRows + wave * kLoadsA;
        L.a_base = G.a + (a_blk << 9);
        L.a_step = static_cast<int64_t>(G.lda) << 10;
        const int64_t a_left = (static_cast<int64_t>(G.k / kBlkCols) * G.lda - a_blk) << 10;
        L.a_bytes = static_cast<uint32_t>(a_left < 0 ? 0 : (a_left > 0x7fffff00ll ? 0x7fffff00ll : a_left));
        L.a_cur = reinterpret_cast<const char*>(L.a_base);
        L.a_left = L.a_bytes;
        L.a_dec = static_cast<uint32_t>(L.a_step > 0x7fffff00ll ? 0x7fffff00ll : L.a_step);
#pragma unroll
        for (int i = 0; i < kLoadsA; ++i) L.voff_a[i] = static_cast<uint32_t>(i * kBlkBytes + lane * 16);
      }
    } else {
      const int rows_a = G.m - row0 < BM ? G.m - row0 : BM;
      const int rows_b = G.n - col0 < kTileN ? G.n - col0 : kTileN;
      L.a_step = L.b_step = 0;
      // K-major operand: load instruction q of the slot (1 KiB of LDS) holds 1024 / row_bytes rows of K; the lane's
      // 16-byte LDS position p = 64 q + lane is chunk p % chunks of row p / chunks, which takes the matrix chunk
      // whose 64-byte segment index is XORed with (row & 3).  Columns past the matrix edge read whatever follows
      // (the next row, or zero past the end): they only reach output rows / columns that are never stored.
      // Rows past K are out of the descriptor's range and read as zero.
      auto k_major_voff = [&](int q, int chunks, int ld) {
        const int pos = 64 * q + lane;
        const int krow = pos / chunks, c = pos % chunks;
        const int src_chunk = ((((c >> 2) ^ (krow & 3)) << 2) | (c & 3));
        return static_cast<uint32_t>(krow) * static_cast<uint32_t>(ld) * 2u + static_cast<uint32_t>(src_chunk) * 16u;
      };
      if constexpr (KA) {
        L.a_base = G.a + row0;
        const int64_t left = (static_cast<int64_t>(G.k) * G.lda - row0) * 2;
        L.a_bytes = static_cast<uint32_t>(left < 0 ? 0 : left);
        L.a_step = static_cast<int64_t>(G.lda) * 2;  // bytes per K row
#pragma unroll
        for (int i = 0; i < kLoadsA; ++i) L.voff_a[i] = k_major_voff(wave * kLoadsA + i, BM / 8, G.lda);
      } else {
        L.a_base = G.a + static_cast<int64_t>(row0) * G.lda;
        L.a_bytes = static_cast<uint32_t>(rows_a) * G.lda * 2u;
        if constexpr (kPA) {
          const uint32_t row_off = static_cast<uint32_t>(wave * kLoadRowsA + pl_row) * G.lda * 2u;
          L.voff_a[0] = row_off + pair_chunk_even * 16u;
          L.voff_a[1] = row_off + pair_chunk_odd * 16u;
          L.pitch8_a = 16u * static_cast<uint32_t>(G.lda);
        } else {
#pragma unroll
          for (int i = 0; i < kLoadsA; ++i) L.voff_a[i] = static_cast<uint32_t>(ld_row0 + 16 * i) * G.lda * 2u + ld_chunk * 16u;
        }
      }
      if constexpr (KB) {
        L.b_base = b_src + col0;
        const int64_t left = (static_cast<int64_t>(G.k) * G.ldb - col0) * 2;
        L.b_bytes = static_cast<uint32_t>(left < 0 ? 0 : left);
        L.b_step = static_cast<int64_t>(G.ldb) * 2;
#pragma unroll
        for (int i = 0; i < kLoadsB; ++i) L.voff_b[i] = k_major_voff(b_wave * kLoadsB + i, BN / 8, G.ldb);
      } else {
        L.b_base = b_src + static_cast<int64_t>(col0) * G.ldb;
        L.b_bytes = static_cast<uint32_t>(rows_b) * G.ldb * 2u;
        if constexpr (kPair) {
          const uint32_t row_off = static_cast<uint32_t>(b_wave * kLoadRowsB + pl_row) * G.ldb * 2u;
          L.voff_b[0] = row_off + pair_chunk_even * 16u;
          L.voff_b[1] = row_off + pair_chunk_odd * 16u;
          L.pitch8_b = 16u * static_cast<uint32_t>(G.ldb);
        } else {
          const int b_ld_row0 = b_wave * kLoadRowsB + (lane >> 2);
#pragma unroll
          for (int i = 0; i < kLoadsB; ++i) L.voff_b[i] = static_cast<uint32_t>(b_ld_row0 + 16 * i) * G.ldb * 2u + ld_chunk * 16u;
        }
      }
    }
  };

  // One K step of global -> LDS for this wave: rows [wave*64, +64) of the A slot, [wave*kLoadRowsB, +kLoadRowsB) of B.
  // The A half goes out right after the barrier that frees the slot, the B half one MFMA group later (spreading
  // the loads keeps the CU's L2 port, 64 bytes per clock, from backing up into the wave's in-order issue);
  // `Pending` carries what the B half needs across that gap, which may include a change of tile.
  struct Pending {
    __amdgpu_buffer_rsrc_t rb;
    uint32_t voff_b[kPB ? 2 : kLoadsB];
    uint32_t pitch8_b;  // paired slots
  };
  // Paired slots: the loads of K steps ks and ks + 1 (ks even) of this wave's rows, A here and B through `Pending`.
  auto issue_pair_a = [&](Loader& L, int ks, unsigned char* pa, Pending& P) {
    const int k0 = ks * BK;
    const uint32_t adv = 2u * static_cast<uint32_t>(k0);
    // as in issue_a: the base advances along K and keeps the absolute end of the readable range, so rows past the
    // matrix read as zero; K chunks at or past the row end are pushed out of range lane by lane
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(L.a_base + k0, L.a_bytes > adv ? L.a_bytes - adv : 0u);
    const bool k_tail = k0 + 2 * BK > L.K;
    const uint32_t oob_even = (k_tail && k0 + pair_chunk_even * 8 >= L.K) ? 0x80000000u : 0u;
    const uint32_t oob_odd = (k_tail && k0 + pair_chunk_odd * 8 >= L.K) ? 0x80000000u : 0u;
    if constexpr (kPB) {
      P.rb = make_rsrc(L.b_base + k0, L.b_bytes > adv ? L.b_bytes - adv : 0u);
      P.voff_b[0] = L.voff_b[0] | oob_even;
      P.voff_b[1] = L.voff_b[1] | oob_odd;
      P.pitch8_b = L.pitch8_b;
    }
    const uint32_t va_even = L.voff_a[0] | oob_even, va_odd = L.voff_a[1] | oob_odd;
#pragma unroll
    for (int i = 0; i < kPairLoadsA; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, LDS_PTR(pa + (wave * kPairLoadsA + i) * 1024), 16,
                                               ((i & 1) ? va_odd : va_even) + static_cast<uint32_t>(i) * L.pitch8_a, 0, 0, 0);
  };
  auto issue_pair_b = [&](const Pending& P, unsigned char* pb) {
#pragma unroll
    for (int i = 0; i < kPairLoadsB; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(P.rb, LDS_PTR(pb + (wave * kPairLoadsB + i) * 1024), 16,
                                               P.voff_b[i & 1] + static_cast<uint32_t>(i) * P.pitch8_b, 0, 0, 0);
  };
  auto issue_a = [&](Loader& L, int ks, unsigned char* sa, Pending& P) {
    __amdgpu_buffer_rsrc_t ra;
    uint32_t oob = 0;
    if constexpr (TILED_IN) {
      // steps past K (ring padding) and blocks past the end of the matrix read as zero through the bounds check
      const bool real = ks * BK < L.K;
      P.rb = make_rsrc(L.b_cur, real ? L.b_left : 0u);
      // on to the next K step.  The byte counts are clamped for huge matrices; a clamped count is far above what
      // one step reads and stays as it is.
      L.b_cur += L.b_step;
      if (L.b_left != 0x7fffff00u) L.b_left = L.b_left > L.b_dec ? L.b_left - L.b_dec : 0u;
      if constexpr (AROWS) {  // token rows: the base advances along K and keeps the absolute end of the readable range
        const uint32_t adv = 2u * static_cast<uint32_t>(ks * BK);
        ra = make_rsrc(L.a_base + ks * BK, real && L.a_bytes > adv ? L.a_bytes - adv : 0u);
      } else {
        ra = make_rsrc(L.a_cur, real ? L.a_left : 0u);
        L.a_cur += L.a_step;
        if (L.a_left != 0x7fffff00u) L.a_left = L.a_left > L.a_dec ? L.a_left - L.a_dec : 0u;
      }
    } else {
      const int k0 = ks * BK;
      // advancing the base keeps the absolute end of the readable range, so rows past the matrix read as zero;
      // K chunks at or past the row end are pushed out of range per lane (this also zero-fills padding steps).
      // A K-major operand advances by whole rows of K instead, and its rows past K are past the end by themselves.
      const uint32_t adv = 2u * static_cast<uint32_t>(k0);
      if constexpr (KA) {
        const int64_t da = L.a_step * k0;
        ra = make_rsrc(reinterpret_cast<const char*>(L.a_base) + da, L.a_bytes > da ? static_cast<uint32_t>(L.a_bytes - da) : 0u);
      } else {
        ra = make_rsrc(L.a_base + k0, L.a_bytes > adv ? L.a_bytes - adv : 0u);
      }
      if constexpr (KB) {
        const int64_t db = L.b_step * k0;
        P.rb = make_rsrc(reinterpret_cast<const char*>(L.b_base) + db, L.b_bytes > db ? static_cast<uint32_t>(L.b_bytes - db) : 0u);
      } else {
        P.rb = make_rsrc(L.b_base + k0, L.b_bytes > adv ? L.b_bytes - adv : 0u);
      }
      const bool k_tail = k0 + BK > L.K;
      oob = (k_tail && k0 + ld_chunk * 8 >= L.K) ? 0x80000000u : 0u;
    }
    const uint32_t oob_a = KA ? 0u : oob, oob_b = KB ? 0u : oob;
    if constexpr (!kPB) {
#pragma unroll
      for (int i = 0; i < kLoadsB; ++i) P.voff_b[i] = L.voff_b[i] | oob_b;
    }
    if constexpr (!kPA) {  // (A in pairs: this call only prepares the step's B descriptor)
#pragma unroll
      for (int i = 0; i < kLoadsA; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, LDS_PTR(sa + (wave * kLoadRowsA + 16 * i) * kRowBytes), 16,
                                                 L.voff_a[i] | oob_a, 0, 0, 0);
    }
  };
  auto issue_b = [&](const Pending& P, unsigned char* sb) {
#pragma unroll
    for (int i = 0; i < kLoadsB; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(P.rb, LDS_PTR(sb + (wave * kLoadRowsB + 16 * i) * kRowBytes), 16,
                                               P.voff_b[i], 0, 0, 0);
  };

  // Fused launch, consumer: the B half of K step `s` of a tile that has not started yet (s < kStages), leaving the
  // loader's running values alone.
  auto issue_b_ahead = [&](const Loader& L, int s, unsigned char* sb) {
    uint32_t left = L.b_left;
    for (int i = 0; i < s; ++i)
      if (left != 0x7fffff00u) left = left > L.b_dec ? left - L.b_dec : 0u;
    Pending P;
    P.rb = make_rsrc(L.b_cur + s * L.b_step, s * BK < L.K ? left : 0u);
#pragma unroll
    for (int i = 0; i < kLoadsB; ++i) P.voff_b[i] = L.voff_b[i];
    issue_b(P, sb);
  };
  // Fused launch: what this workgroup wrote for row block `rb` is in memory (its stores are write-through and every
  // wavefront has waited for its own before the barrier); one lane counts it.
  auto count_done = [&](int* counters, int rb) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    __syncthreads();
    if (tid == 0)
      __hip_atomic_fetch_add(counters + rb * kFusedCounterStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // Fused launch: wait (bounded) until counters[rb] has reached `need`, and take a number among the workgroups that
  // get past this wait (`before`: how many were past it already; the answer travels while the tile is computed).
  // No cache is invalidated afterwards: the launch began with clean caches, and no line of what the wait is for is
  // read anywhere before it is complete (whole cache lines belong to one writer), so no cache can hold an older
  // version of it.
  auto wait_for_count = [&](const int* counters, int* passed, int rb, int need, int& before) {
    if (tid == 0) {
      const int* flag = counters + rb * kFusedCounterStride;
      const long long start = __builtin_amdgcn_s_memrealtime();
      while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < need) {
        if (static_cast<long long>(__builtin_amdgcn_s_memrealtime()) - start > kFusedWaitTicks) {
          __hip_atomic_store(fs.error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      before = __hip_atomic_fetch_add(passed + rb * kFusedCounterStride, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    barrier_no_fence();  // (no wait for the counter's answer here)
  };
  // ... and once the tile is done: the workgroup that was the last of its row block to get past the wait (everything
  // the wait was for is done, and every other waiter is past its wait as well) leaves the two counters at zero for
  // the next launch
  auto clear_if_last = [&](int* counters, int* passed, int rb, int before, int waiters) {
    if (tid == 0 && before == waiters - 1) {
      __hip_atomic_store(counters + rb * kFusedCounterStride, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(passed + rb * kFusedCounterStride, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  // Fused launch, consumer, wavefronts that issue no loads: while the workgroup waits for its row block they pull
  // a share of the PRODUCERS' weights through this XCD's L2, so that weights which come from HBM (every layer of a
  // model has its own) are on their way before the producers' ring, four K steps deep, asks for them.  Workgroup c
  // of the consumers sits on the XCD of producer workgroup c and takes that producer's tile: the K steps
  // k = tm (mod kGroupM) of its gate and up column blocks (the producers of an XCD that share a column tile are the
  // kGroupM tile rows of a patch).  The loads are LDS-direct into the still unused first A slot and are waited for
  // before the barrier that ends the wait.  fs.warm_b is null when the host expects the weights in the caches.
  bool warm_pending = true;
  auto warm_producer_weights = [&]() {
    if constexpr (ROLE == 2) {
      const int total_g = tiles_m[0] * fs.need[0] + tiles_m[1] * fs.need[1];
      TileCoord tg;
      if (wg < total_g && map_tile(wg, total_g, tiles_m, fs.need, tg)) {
        const int e = tg.group;
        static_assert(TS::kWaves - kLoadWaves == 4, "two wavefronts per matrix, each every other K step of the share");
        const int q = wave - kLoadWaves;  // 0 .. 3: matrix q & 1, half q >> 1 of the share
        const __bf16* base = fs.warm_b[e][q & 1];
        if (base != nullptr) {
          const int ldb = fs.warm_ldb[e];
          const int nkb = fs.warm_k / kBlkCols;
          const int64_t bytes = (static_cast<int64_t>(nkb) * ldb) << 10;
          if (bytes < 0x7fffff00ll) {
            const __amdgpu_buffer_rsrc_t r = make_rsrc(base, static_cast<uint32_t>(bytes));
            unsigned char* dummy = slot_a(0) + q * 1024;
            constexpr int kGuBlocks = TS::BN / 2 / kBlkRows;  // row blocks of a gate/up column tile, per matrix
            const int blk0 = tg.tn * kGuBlocks;
            for (int ks = tg.tm % kGroupM + kGroupM * (q >> 1); ks < nkb; ks += 2 * kGroupM) {
#pragma unroll
              for (int i = 0; i < kGuBlocks; ++i) {
                const uint32_t off = static_cast<uint32_t>((static_cast<int64_t>(ks) * ldb + blk0 + i) << 10) + lane * 16;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(r, LDS_PTR(dummy), 16, off, 0, 0, 0);
              }
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
          }
        }
      }
    }
  };
  int passed_before = 0;

  f32x16 acc[FM][FN];
  bf16x8 fa[2][FM], fb[2][FN];  // two fragment sets: one feeds the MFMAs while the other is being read from LDS

  // Fragments are read in the order the MFMAs (A-major: all B blocks for A block 0, then A block 1, ...) first
  // need them: A0, every B, then the other A blocks.
  // K-major slot: K values [8 lhi, +8) of step half kk for the lane's column of 32-column block `blk` (counted
  // from the wave's first block): two transposing reads of four rows each.
  auto read_k_major = [&](const unsigned char* slot, int lane_base, int row_bytes, int blk, int kk) {
    const unsigned char* at = slot + (lane_base ^ (blk << 6)) + 16 * kk * row_bytes;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_TR_PTR(at));
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_TR_PTR(at + 4 * row_bytes));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto read_a = [&](const unsigned char* sa, int i, int kk) {
    if constexpr (KA) return read_k_major(sa, tr_base_a, BM * 2, i, kk);
    else if constexpr (kPA) return *reinterpret_cast<const bf16x8*>(sa + a_pair_off + i * 32 * 128 + frag_off[kk]);
    else return *reinterpret_cast<const bf16x8*>(sa + a_row_off + i * 32 * kRowBytes + frag_off[kk]);
  };
  auto read_b = [&](const unsigned char* sb, int j, int kk) {
    if constexpr (KB) return read_k_major(sb, tr_base_b, BN * 2, j, kk);
    else if constexpr (kPB) return *reinterpret_cast<const bf16x8*>(sb + b_row(j) * 128 + pair_lane_off + frag_off[kk]);
    else return *reinterpret_cast<const bf16x8*>(sb + b_row(j) * kRowBytes + b_lane_off + frag_off[kk]);
  };
  auto read_frags = [&](const unsigned char* sa, const unsigned char* sb, int kk, int set) {
    fa[set][0] = read_a(sa, 0, kk);
#pragma unroll
    for (int j = 0; j < FN; ++j) fb[set][j] = read_b(sb, j, kk);
#pragma unroll
    for (int i = 1; i < FM; ++i) fa[set][i] = read_a(sa, i, kk);
  };
  auto mma = [&](int set) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int jj = 0; jj < FN; ++jj) {
        const int j = jj;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
      }
  };
  // Scheduling hints.  Before the barrier: the LDS reads of the other fragment set and the B half of the previous
  // slot's refill go out among the first half of this group's MFMAs; the second half covers the read latency, so
  // the wait in front of the barrier finds the reads done.
  auto schedule_before_barrier = [&](auto with_loads) {
    constexpr int kB = decltype(with_loads)::value ? kLoadsB : 0;
    constexpr int kMfma = FM * FN, kReads = FM * (KA ? 2 : 1) + FN * (KB ? 2 : 1);
    constexpr int kCarry = kMfma / 2;                              // MFMAs that carry other instructions
    constexpr int kReadsPer = (kReads + kCarry - 1) / kCarry;      // LDS reads per carrying MFMA
    constexpr int kLoadEvery = kB > 0 && kCarry / kB > 0 ? kCarry / kB : 1;
#pragma unroll
    for (int m = 0; m < kCarry; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x100, kReadsPer, 0);
      if (m % kLoadEvery == 0 && m / kLoadEvery < kB) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kMfma - kCarry, 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  // After the barrier: the A half of the refill and the next slot's fragment reads are spread over the whole group.
  auto schedule_after_barrier = [&](auto with_loads) {
    constexpr int kA = decltype(with_loads)::value ? kLoadsA : 0;
    constexpr int kMfma = FM * FN, kReads = FM * (KA ? 2 : 1) + FN * (KB ? 2 : 1);
    constexpr int kReadEvery = kMfma / kReads > 0 ? kMfma / kReads : 1;
    constexpr int kReadsPer = kReads * kReadEvery > kMfma ? (kReads + kMfma - 1) / kMfma : 1;
    constexpr int kLoadEvery = kA > 0 && kMfma / kA > 0 ? kMfma / kA : 1;
#pragma unroll
    for (int m = 0; m < kMfma; ++m) {
      if (m % kLoadEvery == 0 && m / kLoadEvery < kA) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      if (m % kReadEvery == 0 && m / kReadEvery * kReadsPer < kReads) __builtin_amdgcn_sched_group_barrier(0x100, kReadsPer, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // One K step on slot (sa, sb); (sa_n, sb_n) is the next slot of the ring and sb_p the previous one.  On entry
  // fragment set 0 holds kk = 0 of this slot.  After the barrier every wave has finished reading this slot, so its
  // refill with the K step kStages ahead in the load stream (step `ld_ks` of tile `L`) starts at once: the A half
  // here, the B half in the next step's first group.  The next slot's data was issued kStages - 1 steps ago.
  // A wavefront that does not load runs the same step without the load instructions (and its counted wait passes
  // at once: it has no loads in flight).
  Pending pend;
  auto k_step_as = [&](auto with_loads, Loader& L, int ld_ks, unsigned char* sa, unsigned char* sb, unsigned char* sa_n,
                       unsigned char* sb_n, unsigned char* sb_p) {
    constexpr bool LD = decltype(with_loads)::value;
    read_frags(sa, sb, 1, 1);
    if constexpr (LD) issue_b(pend, sb_p);
    mma(0);
    schedule_before_barrier(with_loads);
    // my LDS reads have returned; of my loads at most the kStages - 2 youngest K steps' worth are still in flight,
    // i.e. the next slot is complete
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(LD ? (kStages - 2) * kLoadsPerStep : 63, 0));
    barrier_no_fence();
    if constexpr (LD) issue_a(L, ld_ks, sa, pend);
    read_frags(sa_n, sb_n, 0, 0);
    mma(1);
    schedule_after_barrier(with_loads);
  };
  // The same step on paired slots (step S of a ring round; slots 0, 1 are pair 0, slots 2, 3 pair 1).  A pair is
  // free once its odd slot has been read, i.e. after the barrier of steps 1 and 3: its A refill (the K steps one ring
  // round ahead) goes out there, its B refill at the start of the following step, and everything must have landed
  // by the barrier two steps on, which is the only load still in flight then -- the counted wait becomes vmcnt(0) on
  // odd steps and none on even ones.
  auto schedule_pair = [&](auto n_before, auto n_after) {
    constexpr int kB = decltype(n_before)::value, kA = decltype(n_after)::value;
    constexpr int kMfma = FM * FN, kReads = FM + FN;
    (void)kA;
    constexpr int kCarry = kMfma / 2;
    constexpr int kReadsPer = (kReads + kCarry - 1) / kCarry;
    constexpr int kBd = kB > 0 ? kB : 1;
    constexpr int kLoadEvery = kCarry / kBd > 0 ? kCarry / kBd : 1;
    constexpr int kLoadsPer = kB > kCarry ? (kB + kCarry - 1) / kCarry : 1;
#pragma unroll
    for (int m = 0; m < kCarry; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x100, kReadsPer, 0);
      if (kB > 0 && m % kLoadEvery == 0 && m / kLoadEvery * kLoadsPer < kB) __builtin_amdgcn_sched_group_barrier(0x020, kLoadsPer, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kMfma - kCarry, 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto schedule_pair_after = [&](auto n_after) {
    constexpr int kA = decltype(n_after)::value;
    constexpr int kMfma = FM * FN, kReads = FM * (KA ? 2 : 1) + FN * (KB ? 2 : 1);
    constexpr int kReadEvery = kMfma / kReads > 0 ? kMfma / kReads : 1;
    constexpr int kReadsPer = kReads * kReadEvery > kMfma ? (kReads + kMfma - 1) / kMfma : 1;
    constexpr int kAd = kA > 0 ? kA : 1;
    constexpr int kLoadEvery = kMfma / kAd > 0 ? kMfma / kAd : 1;
    constexpr int kLoadsPer = kA > kMfma ? (kA + kMfma - 1) / kMfma : 1;
#pragma unroll
    for (int m = 0; m < kMfma; ++m) {
      if (kA > 0 && m % kLoadEvery == 0 && m / kLoadEvery * kLoadsPer < kA) __builtin_amdgcn_sched_group_barrier(0x020, kLoadsPer, 0);
      if (m % kReadEvery == 0 && m / kReadEvery * kReadsPer < kReads) __builtin_amdgcn_sched_group_barrier(0x100, kReadsPer, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto k_step_pair = [&](auto with_loads, auto step_c, Loader& L, int ld_ks) {
    constexpr bool LD = decltype(with_loads)::value;
    constexpr int S = decltype(step_c)::value;
    constexpr bool kOdd = (S & 1) != 0;
    read_frags(slot_a(S), slot_b(S), 1, 1);
    if constexpr (LD && !kOdd) issue_pair_b(pend, S == 0 ? s_pb1 : s_pb0);
    mma(0);
    schedule_pair(std::integral_constant<int, (LD && !kOdd) ? kPairLoadsB : 0>{}, std::integral_constant<int, 0>{});
    __builtin_amdgcn_s_waitcnt(waitcnt_imm((LD && kOdd) ? 0 : 63, 0));
    barrier_no_fence();
    if constexpr (LD && kOdd) issue_pair_a(L, ld_ks + (S == 1 ? 0 : 2), S == 1 ? s_pa0 : s_pa1, pend);
    read_frags(slot_a((S + 1) % kStages), slot_b((S + 1) % kStages), 0, 0);
    mma(1);
    schedule_pair_after(std::integral_constant<int, (LD && kOdd) ? kPairLoadsA : 0>{});
  };
  // ... and with A alone in pairs (NN).  B keeps the slot-by-slot schedule of k_step_as (the refill of slot S - 1 at
  // the start of step S, its descriptor prepared after the barrier of step S - 1), A the pairs' (after the barrier of
  // odd steps).  In flight behind what the barrier of step S needs: the B refills of the two youngest steps, and on
  // even steps the A pair issued one step ago as well.
  auto k_step_mixed = [&](auto with_loads, auto step_c, Loader& L, int ld_ks) {
    constexpr bool LD = decltype(with_loads)::value;
    constexpr int S = decltype(step_c)::value;
    constexpr bool kOdd = (S & 1) != 0;
    read_frags(slot_a(S), slot_b(S), 1, 1);
    if constexpr (LD) issue_b(pend, slot_b((S + kStages - 1) % kStages));
    mma(0);
    schedule_before_barrier(with_loads);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(LD ? (kOdd ? 2 * kLoadsB : 2 * kLoadsB + kPairLoadsA) : 63, 0));
    barrier_no_fence();
    if constexpr (LD) {
      issue_a(L, ld_ks + S, nullptr, pend);
      if constexpr (kOdd) issue_pair_a(L, ld_ks + S - 1, S == 1 ? s_pa0 : s_pa1, pend);
    }
    read_frags(slot_a((S + 1) % kStages), slot_b((S + 1) % kStages), 0, 0);
    mma(1);
    schedule_pair_after(std::integral_constant<int, (LD && kOdd) ? kPairLoadsA : 0>{});
  };
  // ---- epilogue ------------------------------------------------------------------------------------------
  // Accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 block.  Values
  // are rounded to bf16, paired with the neighbouring column through a lane swap (even lanes keep the even
  // register's row, odd lanes the odd register's row), written to this wave's staging area as dwords, and read
  // back as 16-byte lanes laid out the way the destination wants them.
  unsigned char* stage = s_out + wave * kStageBytes;
  // Stores register pair (r, r+1) of one 32x32 block -- rows srow and srow + 1, column scol of this lane -- into
  // the staging area with row pitch `pitch` bytes.
  auto stage_pair = [&](float v0, float v1, int srow, int scol, int pitch, int odd) {
    // both values are converted at once (low half v0, high half v1) and the pair is swapped with the neighbour;
    // even lane keeps (own v0, neighbour's v0) -> row srow; odd lane (neighbour's v1, own v1) -> row srow + 1.
    // One byte permute picks the two halves: selector bytes 0-3 address `theirs`, 4-7 address `mine`.
    const uint32_t mine = pack_bf16x2(v0, v1);
    const uint32_t theirs = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(mine), 0xB1, 0xF, 0xF, true));
    const uint32_t sel = odd ? 0x07060302u : 0x01000504u;
    const uint32_t packed = __builtin_amdgcn_perm(mine, theirs, sel);
    *reinterpret_cast<uint32_t*>(stage + (srow + odd) * pitch + (scol & ~1) * 2) = packed;
  };

  auto epilogue = [&](const Store& S) {
    // The lane id is laundered through an empty asm so the address arithmetic is redone here each tile instead
    // of being hoisted out of the persistent loop and held in registers across the K loop.
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int el32 = lane_e & 31, elhi = lane_e >> 5, odd = lane_e & 1;
    if constexpr (SWIGLU) {
      // wave output: 128 rows x kOutCols intermediate columns, staged kRound rows at a time
      constexpr int kOutCols = FN / 2 * 32;
      constexpr int kPitch = kOutCols * 2;
      constexpr int kRound = kStageBytes / kPitch;  // rows per round (64 / 32)
      constexpr int kIPerRound = kRound / 32;       // 32-row accumulator blocks per round
      static_assert(kIPerRound >= 1 && FM % kIPerRound == 0, "staging holds whole accumulator blocks");
      // what == 0: the intermediate h; 1 / 2: the gate / up projections themselves, when the caller keeps them
      const int n_what = p.keep_gate != nullptr ? 3 : 1;
      const int64_t keep_off[3] = {0, reinterpret_cast<unsigned char*>(p.keep_gate) - reinterpret_cast<unsigned char*>(p.g[0].c),
                                   reinterpret_cast<unsigned char*>(p.keep_up) - reinterpret_cast<unsigned char*>(p.g[0].c)};
#pragma unroll
      for (int round = 0; round < FM / kIPerRound; ++round) {
        for (int what = 0; what < n_what; ++what) {
#pragma unroll
          for (int ii = 0; ii < kIPerRound; ++ii) {
            const int i = round * kIPerRound + ii;
#pragma unroll
            for (int j = 0; j < FN / 2; ++j) {
#pragma unroll
              for (int r = 0; r < 16; r += 2) {
                float h[2];
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                  // eager bf16 evaluation of act_fn(gate) * up (act.py:80-82): gate, up, silu(gate) and the
                  // product are each rounded to bf16
                  const uint32_t gu = pack_bf16x2(acc[i][j][r + q], acc[i][j + FN / 2][r + q]);  // one convert for both
                  const float g = __uint_as_float(gu << 16);
                  const float u = __uint_as_float(gu & 0xffff0000u);
                  if (what == 0) {
                    const float sg = round_bf16(g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)));
                    h[q] = sg * u;
                  } else {
                    h[q] = what == 1 ? g : u;
                  }
                }
                const int srow = ii * 32 + 8 * (r >> 2) + 4 * elhi + (r & 3);
                stage_pair(h[0], h[1], srow, j * 32 + el32, kPitch, odd);
              }
            }
          }
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
          // kRound rows x kOutCols columns = (kRound / 16) row blocks x (kOutCols / 32) column blocks of the tiled
          // intermediate, 1 KiB each; one store instruction per block: lane -> (row lane/4, slot lane%4) holding
          // chunk slot ^ ((row >> 2) & 3)
          const int r16 = lane_e >> 2, slot = lane_e & 3, chunk = slot ^ ((r16 >> 2) & 3);
#pragma unroll
          for (int rbl = 0; rbl < kRound / 16; ++rbl) {
#pragma unroll
            for (int kbl = 0; kbl < kOutCols / 32; ++kbl) {
              const u32x4 v =
                  *reinterpret_cast<const u32x4*>(stage + (rbl * 16 + r16) * kPitch + (kbl * 32 + chunk * 8) * 2);
              const int row = wm * (FM * 32) + round * kRound + rbl * 16;  // first row of the block inside the tile
              const int col = wn * kOutCols + kbl * 32;                     // first column of the block inside the tile
              // rows past the expert's last row are padding of the tiled matrix: harmless to write, never read
              if (col < S.cols_left) {
                unsigned char* dst = reinterpret_cast<unsigned char*>(S.c_base) + keep_off[what] +
                                     ((static_cast<int64_t>(col / kBlkCols) * S.ldc + row / kBlkRows) << 10);
                if constexpr (ROLE == 1) {
                  // fused launch: written through to memory (agent-scope store), so that the tile is visible to
                  // the other XCDs once the stores have completed, without a write-back of this XCD's L2
                  __builtin_amdgcn_raw_buffer_store_b128(v, make_rsrc(dst, kBlkBytes), lane_e * 16, 0, 16 /* sc1 */);
                } else {
                  *reinterpret_cast<u32x4*>(dst + lane_e * 16) = v;
                }
              }
            }
          }
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));  // staging is rewritten by the next round
        }
      }
    } else {
      if constexpr (MODE == kQkvRope || MODE == kQkvRopeFull) {
        // Bias and rotary embedding on the accumulators, before they are staged.  A wavefront's 128 columns are one
        // head; channel d of the head sits in block d / 32 at lane d % 32, so its rotation partner d +/- 64 is two
        // blocks away in the same lane.  Evaluated like eager bf16 code: the projection (with its bias) rounded once,
        // then q * cos + rotate_half(q) * sin with each product and the sum rounded (vl.py:771-772).
        static_assert(FN == 4, "a wavefront covers whole heads of 128 channels");
        const int col_w = S.col0 + wn * 128;  // first output column of this wavefront's head
        const bool live = wn * 128 < S.cols_left;
        float bias_v[4] = {0.f, 0.f, 0.f, 0.f};
        if (p.bias != nullptr && live) {
#pragma unroll
          for (int j = 0; j < 4; ++j) bias_v[j] = static_cast<float>(p.bias[col_w + j * 32 + el32]);
        }
        const bool rotate = live && col_w < p.rope_cols;  // wave-uniform: q and k heads rotate, v heads do not
        if constexpr (MODE == kQkvRope) {  // channels d and d + 64 share a table entry (64 per token)
#pragma unroll
          for (int i = 0; i < FM; ++i) {
            // cos | sin of this lane's channels 32 jp + lane % 32 (shared with the channel 64 further) for its 16 rows:
            // all 32 loads go out before the first is used
            uint32_t cs[16][2];
            if (rotate) {
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int row = wm * (FM * 32) + i * 32 + 8 * (r >> 2) + 4 * elhi + (r & 3);
                const bool in = row < S.rows;
                const uint32_t* t = p.rope_table + static_cast<int64_t>(S.row0 + (in ? row : 0)) * 64 + el32;
                cs[r][0] = t[0];
                cs[r][1] = t[32];
              }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
#pragma unroll
              for (int jp = 0; jp < 2; ++jp) {
                const float lo = round_bf16(acc[i][jp][r] + bias_v[jp]);
                const float hi = round_bf16(acc[i][jp + 2][r] + bias_v[jp + 2]);
                if (rotate) {
                  const float c = __uint_as_float(cs[r][jp] << 16), sn = __uint_as_float(cs[r][jp] & 0xffff0000u);
                  acc[i][jp][r] = round_bf16(lo * c) - round_bf16(hi * sn);
                  acc[i][jp + 2][r] = round_bf16(hi * c) + round_bf16(lo * sn);
                } else {
                  acc[i][jp][r] = lo;
                  acc[i][jp + 2][r] = hi;
                }
              }
            }
          }
        } else {
          // one table entry per channel (128 per token): the same walk, one half of the channel pairs at a time (32
          // entries in flight)
#pragma unroll
          for (int i = 0; i < FM; ++i) {
#pragma unroll
            for (int jp = 0; jp < 2; ++jp) {
              uint32_t cs[16][2];  // [row][0]: channel 32 jp + lane % 32, [1]: the channel 64 further
              if (rotate) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                  const int row = wm * (FM * 32) + i * 32 + 8 * (r >> 2) + 4 * elhi + (r & 3);
                  const bool in = row < S.rows;
                  const uint32_t* t = p.rope_table + static_cast<int64_t>(S.row0 + (in ? row : 0)) * 128 + jp * 32 + el32;
                  cs[r][0] = t[0];
                  cs[r][1] = t[64];
                }
              }
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const float lo = round_bf16(acc[i][jp][r] + bias_v[jp]);
                const float hi = round_bf16(acc[i][jp + 2][r] + bias_v[jp + 2]);
                if (rotate) {
                  const float c_lo = __uint_as_float(cs[r][0] << 16), s_lo = __uint_as_float(cs[r][0] & 0xffff0000u);
                  const float c_hi = __uint_as_float(cs[r][1] << 16), s_hi = __uint_as_float(cs[r][1] & 0xffff0000u);
                  acc[i][jp][r] = round_bf16(lo * c_lo) - round_bf16(hi * s_lo);
                  acc[i][jp + 2][r] = round_bf16(hi * c_hi) + round_bf16(lo * s_hi);
                } else {
                  acc[i][jp][r] = lo;
                  acc[i][jp + 2][r] = hi;
                }
              }
            }
          }
        }
      }
      // wave output: 128 rows x kOutCols columns row-major, staged kRound rows at a time
      constexpr int kOutCols = FN * 32;
      constexpr int kPitch = kOutCols * 2;
      constexpr int kRound = kStageBytes / kPitch;  // 32 / 16 rows
      constexpr int kParts = 32 / kRound;           // rounds per 32-row accumulator block
      static_assert(kParts == 1 || kParts == 2, "a round is a whole or half accumulator block");
      constexpr int kLanesPerRow = kPitch / 16, kRowsPerStore = 64 / kLanesPerRow;
#pragma unroll
      for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int part = 0; part < kParts; ++part) {
          // a row is kPitch bytes = kLanesPerRow lanes; one store instruction writes kRowsPerStore rows
          const int rl = lane_e / kLanesPerRow, cc = (lane_e % kLanesPerRow) * 8;
          const int col = wn * kOutCols + cc;
          constexpr int kStores = kRound / kRowsPerStore;
          int out_row[kStores];
          u32x4 resv[kStores];
#pragma unroll
          for (int q = 0; q < kStores; ++q) {
            const int row = wm * (FM * 32) + i * 32 + part * kRound + q * kRowsPerStore + rl;
            out_row[q] = row;
            if constexpr (MODE == kDown) {
              // scatter: the row ids of the round (and the residual's chunks) are fetched together, ahead of the
              // staging writes and reads
              if (S.row_id != nullptr && row < S.rows) out_row[q] = S.row_id[row];
            }
          }
          if constexpr (MODE == kDown || MODE == kGeneric) {
            if (S.res != nullptr) {
#pragma unroll
              for (int q = 0; q < kStores; ++q) {
                const int row = wm * (FM * 32) + i * 32 + part * kRound + q * kRowsPerStore + rl;
                resv[q] = u32x4{0u, 0u, 0u, 0u};
                if (row < S.rows && col < S.cols_left)
                  resv[q] = *reinterpret_cast<const u32x4*>(S.res + static_cast<int64_t>(out_row[q]) * S.ldc + col);
              }
            }
          }
#pragma unroll
          for (int j = 0; j < FN; ++j) {
#pragma unroll
            for (int rr = 0; rr < 16 / kParts; rr += 2) {
              const int r = part * (16 / kParts) + rr;  // half blocks: registers 0..7 are rows 0..15, 8..15 rows 16..31
              const int srow = 8 * (r >> 2) + 4 * elhi + (r & 3) - part * kRound;
              stage_pair(acc[i][j][r], acc[i][j][r + 1], srow, j * 32 + el32, kPitch, odd);
            }
          }
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
#pragma unroll
          for (int q = 0; q < kStores; ++q) {
            const int srow = q * kRowsPerStore + rl;
            u32x4 v = *reinterpret_cast<const u32x4*>(stage + srow * kPitch + cc * 2);
            const int row = wm * (FM * 32) + i * 32 + part * kRound + srow;
            if constexpr (MODE == kDown || MODE == kGeneric) {
              if (S.res != nullptr) {  // bf16(y) + bf16(residual), summed in fp32 and rounded once, like the eager add
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                  const float lo = __builtin_bit_cast(float, v[w] << 16) + __builtin_bit_cast(float, resv[q][w] << 16);
                  const float hi = __builtin_bit_cast(float, v[w] & 0xFFFF0000u) +
                                   __builtin_bit_cast(float, resv[q][w] & 0xFFFF0000u);
                  v[w] = pack_bf16x2(lo, hi);
                }
              }
            }
            if (row < S.rows && col < S.cols_left)
              *reinterpret_cast<u32x4*>(S.c_base + static_cast<int64_t>(out_row[q]) * S.ldc + col) = v;
          }
          __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
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
  int next_t = wg;
  auto next_tile = [&](TileCoord& tc) {
    bool have = false;
    if (kIsTail && p.split == 2) {
      for (; next_t < pieces && !have; next_t += n_wg) {
        const int piece = next_t % (kSubM * kSubN);
        tile_coords(split_at + next_t / (kSubM * kSubN), big_m, big_n, tc);
        tc.tm = kSubM * tc.tm + piece / kSubN;
        tc.tn = kSubN * tc.tn + piece % kSubN;
        // pieces past a ragged last row / column of tiles are empty
        have = tc.tm < (tc.group ? tiles_m[1] : tiles_m[0]) && tc.tn < (tc.group ? tiles_n[1] : tiles_n[0]);
      }
      return have;
    }
    for (; next_t < padded && !have; next_t += n_wg) have = map_tile(next_t, total, tiles_m, tiles_n, tc);
    return have;
  };
  TileCoord tc;
  bool have = next_tile(tc);
  if (!have) return;
  // The whole tile loop exists in two forms, with and without the load instructions; a wavefront picks its form
  // once (all of them the first, unless only some wavefronts load).
  auto run = [&](auto with_loads) {
    constexpr bool LD = decltype(with_loads)::value;
    Loader L;
    Store S;
    if constexpr (LD) setup_loader(tc, L);
    setup_store(tc, S);
    // Consumer of a fused launch: every tile starts from an empty ring.  The weights of the first ring slots are
    // fetched at once, the intermediate only after the row block's producers have finished; then the ring is as the
    // plain prologue leaves it (the last slot's B half goes out in the first K step), with every load landed.
    auto consumer_prologue = [&]() {
      static_assert(ROLE != 2 || TILED_IN, "the fused launch runs the tiled forms");
      if constexpr (LD) {
#pragma unroll
        for (int s = 0; s + 1 < kStages; ++s) issue_b_ahead(L, s, slot_b(s));
      }
      if constexpr (!LD && ASYM) {
        if (warm_pending) {
          warm_pending = false;
          warm_producer_weights();
        }
      }
      wait_for_count(fs.ready, fs.passed, S.row_block, fs.need[tc.group], passed_before);
      if constexpr (LD) {
#pragma unroll
        for (int s = 0; s < kStages; ++s) issue_a(L, s, slot_a(s), pend);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
      }
    };
    if constexpr (ROLE == 2) {
      consumer_prologue();
    } else if constexpr (LD && kPair) {
      issue_pair_a(L, 0, s_pa0, pend);
      issue_pair_b(pend, s_pb0);
      issue_pair_a(L, 2, s_pa1, pend);  // this pair's B half goes out in the first K step
      // pair 0 must be complete before its first fragments are read: pair 1's A half may remain in flight
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(kPairLoadsA, 15));
    } else if constexpr (LD && kPairAOnly) {
      // in the order the steps keep: A's first pair, B's slots 0 and 1, A's second pair, B's slot 2 (slot 3 goes out in
      // the first K step)
      issue_a(L, 0, nullptr, pend);
      issue_pair_a(L, 0, s_pa0, pend);
      issue_b(pend, slot_b(0));
      issue_a(L, 1, nullptr, pend);
      issue_b(pend, slot_b(1));
      issue_pair_a(L, 2, s_pa1, pend);
      issue_a(L, 2, nullptr, pend);
      issue_b(pend, slot_b(2));
      issue_a(L, 3, nullptr, pend);
      // slot 0 of both operands must be complete: everything behind B's slot 0 may remain in flight
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * kLoadsB + kPairLoadsA, 15));
    } else if constexpr (LD) {
#pragma unroll
      for (int s = 0; s < kStages; ++s) {
        issue_a(L, s, slot_a(s), pend);
        if (s + 1 < kStages) issue_b(pend, slot_b(s));  // the last slot's B half goes out in the first K step
      }
      // slot 0 must be complete before its first fragments are read: the younger loads may remain in flight
      __builtin_amdgcn_s_waitcnt(waitcnt_imm((kStages - 2) * kLoadsPerStep + kLoadsA, 15));
    }
    __syncthreads();
    read_frags(slot_a(0), slot_b(0), 0, 0);

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
          // (a consumer of a fused launch lets the ring run empty: its next tile has a wait of its own in front)
          have = ROLE == 2 ? false : next_tile(tc);
          if (have) {
            if constexpr (LD) setup_loader(tc, L);
            setup_store(tc, S);
          } else if constexpr (LD) {
            L.a_bytes = L.a_left = 0;
            L.b_bytes = L.b_left = 0;
            L.K = 0;
          }
          ld_ks = 0;
        }
        if constexpr (kPairAOnly) {
          k_step_mixed(with_loads, std::integral_constant<int, 0>{}, L, ld_ks);
          k_step_mixed(with_loads, std::integral_constant<int, 1>{}, L, ld_ks);
          k_step_mixed(with_loads, std::integral_constant<int, 2>{}, L, ld_ks);
          k_step_mixed(with_loads, std::integral_constant<int, 3>{}, L, ld_ks);
        } else if constexpr (kPair) {
          k_step_pair(with_loads, std::integral_constant<int, 0>{}, L, ld_ks);
          k_step_pair(with_loads, std::integral_constant<int, 1>{}, L, ld_ks);
          k_step_pair(with_loads, std::integral_constant<int, 2>{}, L, ld_ks);
          k_step_pair(with_loads, std::integral_constant<int, 3>{}, L, ld_ks);
        } else {
#pragma unroll
          for (int s = 0; s < kStages; ++s)
            k_step_as(with_loads, L, ld_ks + s, slot_a(s), slot_b(s), slot_a((s + 1) % kStages), slot_b((s + 1) % kStages),
                      slot_b((s + kStages - 1) % kStages));
        }
      }
      epilogue(done);
      if constexpr (ROLE == 1) count_done(fs.ready, done.row_block);
      if constexpr (ROLE == 2) {
        clear_if_last(fs.ready, fs.passed, done.row_block, passed_before, fs.consumers);
        have = next_tile(tc);
        if (have) {  // (one tile per consumer unless the host's row counts were not the device's)
          if constexpr (LD) setup_loader(tc, L);
          setup_store(tc, S);
          consumer_prologue();
          __syncthreads();
          read_frags(slot_a(0), slot_b(0), 0, 0);
        }
      }
    }
  };
  if constexpr (!ASYM) {
    run(std::true_type{});
  } else {
    if (loads) run(std::true_type{});
    else run(std::false_type{});
  }
#endif
}

template <int MODE, typename TS, bool KA = false, bool KB = false>
__global__ __launch_bounds__(TS::kThreads, TS::kWgPerCu) void dual_gemm_kernel(Params p) {
  dual_gemm_body<MODE, TS, KA, KB, 0>(p, blockIdx.x, gridDim.x, FusedSync{});
}

// The fused FFN launch (see FusedSync): workgroups [0, producers) run the gate/up form on `pg`, the rest the down
// form on `pd`, both in the small tile shape.  `producers` is a multiple of 8, so a workgroup's index among its
// form's workgroups names the same XCD as its index in the grid.  (A workgroup that waits is a consumer, and what
// it waits for belongs to workgroups with lower indices, which never wait: whatever part of the grid is resident,
// the launch makes progress.)
// AROWS: the producers read the token rows (fs.x through fs.gather) in place of the K-tiled activations.
template <bool AROWS>
__global__ __launch_bounds__(SmallTile::kThreads, SmallTile::kWgPerCu) void ffn_fused_kernel(Params pg, Params pd,
                                                                                             FusedSync fs,
                                                                                             int producers) {
  const int wg = blockIdx.x;
  if (wg < producers) dual_gemm_body<kGateUp, SmallTile, false, false, 1, AROWS>(pg, wg, producers, fs);
  else dual_gemm_body<kDown, SmallTile, false, false, 2>(pd, wg - producers, static_cast<int>(gridDim.x) - producers, fs);
}

// ---- plain FMA tiles: any transpose combination, any k --------------------------------------------------------
// Used for what the MFMA kernel does not take: K-major operands of 4 GiB or more.
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
          for (int q = 0; q < 4; ++q) acc[q] = fmaf(s_a[ty + 8 * q][kk], bv, acc[q]);
        }
        __syncthreads();
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = row0 + ty + 8 * q, n = col0 + tx;
        if (m < G.m && n < G.n) {
          __bf16 v = static_cast<__bf16>(acc[q]);
          if (G.add != nullptr) v = static_cast<__bf16>(static_cast<float>(v) + static_cast<float>(G.add[static_cast<int64_t>(m) * G.ldc + n]));
          G.c[static_cast<int64_t>(m) * G.ldc + n] = v;
        }
      }
    }
  }
}

// Row-major [rows, cols] bf16 -> K-tiled (rows padded to 16 with zeros).  One thread per 16-byte chunk.
__global__ __launch_bounds__(256) void pack_tiled_kernel(const u32x4* __restrict__ src, unsigned char* __restrict__ dst,
                                                         int64_t rows, int64_t cols) {
  const int64_t chunks_per_row = cols / 8;
  const int64_t row_blocks = tiled_row_blocks(rows);
  const int64_t n = row_blocks * kBlkRows * chunks_per_row;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t row = i / chunks_per_row, c = i - row * chunks_per_row;
    const u32x4 v = row < rows ? src[i] : u32x4{0, 0, 0, 0};
    *reinterpret_cast<u32x4*>(dst + tiled_chunk_offset(row, c * 8, row_blocks)) = v;
  }
}

// Zeros for the output of an empty contraction (k == 0): a fill kernel rather than a memset node, so that the call
// stays capturable in a HIP graph like every other launch here.  n16 = number of 16-byte chunks.
__global__ __launch_bounds__(256) void zero_fill_kernel(u32x4* __restrict__ dst, int64_t n16) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    dst[i] = u32x4{0, 0, 0, 0};
}

// k_in_rows: both operands are stored with K as the slow dimension, so K needs no alignment
int check_dims(const char* who, int64_t m, int64_t n, int64_t k, bool k_in_rows = false) {
  if (m < 0 || n < 0 || k < 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: negative dimension", who);
  if (m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: dimension exceeds int32", who);
  if (n % 8 != 0 || (k % 8 != 0 && !k_in_rows))
    return fail(WX_ERR_UNSUPPORTED, "%s: n (%lld) and k (%lld) must be multiples of 8", who, static_cast<long long>(n),
                static_cast<long long>(k));
  // 256 rows of one operand must stay addressable through a 31-bit buffer offset
  if (k * 2 * 256 >= (1ll << 31) || n * 2 * 256 >= (1ll << 31)) return fail(WX_ERR_UNSUPPORTED, "%s: row too long", who);
  // the tile list is indexed with 32-bit integers
  if (((m + SmallTile::BM - 1) / SmallTile::BM) * ((n + SmallTile::BN / 2 - 1) / (SmallTile::BN / 2)) >= (1ll << 30))
    return fail(WX_ERR_UNSUPPORTED, "%s: too many tiles", who);
  return WX_OK;
}

// The problem has between `tiles_lo` and `tiles_hi` 256 x 256 tiles (equal when the host knows the row counts).
// When they would occupy at most half of the CUs, the 128 x 128 tile gives four times as many workgroups to spread
// over the chip.  If the bounds fall on both sides of that threshold the choice is made on the device: both
// shapes are launched and the one on the wrong side returns immediately.
// tiles_by_expert: the host's exact 256 x 256 tile counts per expert, or null when only the device knows the row
// split (the bounds are then on the plain sum of the tiles; where they straddle the threshold and the device
// chooses, it chooses by shape_deciding_tiles like the host would).  A launch of large tiles uses the tail split: a
// second launch with 128 x 128 tiles takes the ragged last round when that pays (the row-major op, whose sizes the
// host knows, decides it on the host); when the host cannot tell, both launches are made and the device decides (the
// second returns at once if there is nothing to split).
template <int MODE, bool KA = false, bool KB = false>
int launch_mfma(Params p, int64_t tiles_lo, int64_t tiles_hi, hipStream_t s, const char* who,
                const int64_t* tiles_by_expert = nullptr) {
  const int cus = device_cu_count();
  const int threshold = cus / 2;
  bool small = tiles_lo <= threshold, big = tiles_hi > threshold;
  if (tiles_by_expert != nullptr) {  // the host knows the split: the count that decides is shape_deciding_tiles'
    small = shape_deciding_tiles(tiles_by_expert[0], tiles_by_expert[1], p.g[0].k, p.g[1].k) <= threshold;
    big = !small;
  } else if (!small && tiles_lo <= cus && (2ll * p.g[0].k <= p.g[1].k || 2ll * p.g[1].k <= p.g[0].k)) {
    // at most one round of large tiles, and one expert's tiles may not count: the device has to choose
    small = true;
  }
  p.gate_tiles = threshold;
  p.split = 0;
  p.split_cus = cus;
  if (small) {
    p.gate = big ? 1 : 0;
    hipLaunchKernelGGL((dual_gemm_kernel<MODE, SmallTile, KA, KB>), dim3(cus * SmallTile::kWgPerCu),
                       dim3(SmallTile::kThreads), 0, s, p);
  }
  if (big) {
    p.gate = small ? 2 : 0;
    using Big = BigTileFor<MODE>;
    static_assert(Big::kWgPerCu == 1, "the split counts one large tile per CU and round");
    bool split = (MODE != kGeneric || tiles_by_expert != nullptr) && tiles_hi > cus;
    if (split && tiles_by_expert != nullptr) {
      const int64_t all = tiles_by_expert[0] + tiles_by_expert[1];
      split = all < INT32_MAX && tail_split_point(static_cast<int>(tiles_by_expert[0]), static_cast<int>(tiles_by_expert[1]),
                                                  p.g[0].k, p.g[1].k, cus) != all;
    }
    p.split = split ? 1 : 0;
    hipLaunchKernelGGL((dual_gemm_kernel<MODE, Big, KA, KB>), dim3(cus), dim3(Big::kThreads), 0, s, p);
    if (split) {
      p.split = 2;
      hipLaunchKernelGGL((dual_gemm_kernel<MODE, TailTile, KA, KB>), dim3(cus * TailTile::kWgPerCu),
                         dim3(TailTile::kThreads), 0, s, p);
    }
  }
  return check_launch(who);
}

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace
}  // namespace wx

using namespace wx;

namespace {
int dual_gemm_impl(const void* in0, const void* in1, const void* w0, const void* w1, void* out0, void* out1,
                   const void* add0, const void* add1, int64_t m0, int64_t n0, int64_t k0, int64_t m1, int64_t n1,
                   int64_t k1, int trans_a, int trans_b, wx_stream_t stream);
}

extern "C" int wx_dual_gemm(const void* in0, const void* in1, const void* w0, const void* w1, void* out0, void* out1,
                            int64_t m0, int64_t n0, int64_t k0, int64_t m1, int64_t n1, int64_t k1, int trans_a,
                            int trans_b, wx_stream_t stream) {
  return dual_gemm_impl(in0, in1, w0, w1, out0, out1, nullptr, nullptr, m0, n0, k0, m1, n1, k1, trans_a, trans_b, stream);
}

extern "C" int wx_dual_gemm_add(const void* in0, const void* in1, const void* w0, const void* w1, void* out0,
                                void* out1, const void* add0, const void* add1, int64_t m0, int64_t n0, int64_t k0,
                                int64_t m1, int64_t n1, int64_t k1, int trans_a, int trans_b, wx_stream_t stream) {
  if ((reinterpret_cast<uintptr_t>(add0) | reinterpret_cast<uintptr_t>(add1)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "wx_dual_gemm_add: buffers must be 16-byte aligned");
  return dual_gemm_impl(in0, in1, w0, w1, out0, out1, add0, add1, m0, n0, k0, m1, n1, k1, trans_a, trans_b, stream);
}

namespace {
int dual_gemm_impl(const void* in0, const void* in1, const void* w0, const void* w1, void* out0, void* out1,
                   const void* add0, const void* add1, int64_t m0, int64_t n0, int64_t k0, int64_t m1, int64_t n1,
                   int64_t k1, int trans_a, int trans_b, wx_stream_t stream) {
  const void* adds[2] = {add0, add1};
  gemm_path_reset();
  const bool k_in_rows = trans_a && !trans_b;  // A [k, m] and B [k, n]
  if (int rc = check_dims("wx_dual_gemm", m0, n0, k0, k_in_rows)) return rc;
  if (int rc = check_dims("wx_dual_gemm", m1, n1, k1, k_in_rows)) return rc;
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
    g.a_row0 = 0;
    g.add = static_cast<const __bf16*>(adds[e]);
  }
  p.offsets = nullptr;
  if ((m0 == 0 || n0 == 0) && (m1 == 0 || n1 == 0)) return WX_OK;
  hipStream_t s = as_stream(stream);
  // an empty contraction (k == 0) has zeros as its result: a fill launch writes them and the group leaves the
  // problem, so the other expert still runs on the MFMA kernel (a training batch without action tokens has k == 0
  // in the action expert's weight gradients next to the VL expert's full-size ones)
  for (int e = 0; e < 2; ++e) {
    const int64_t m = dims[e][0], n = dims[e][1];
    if (dims[e][2] != 0 || m <= 0 || n <= 0) continue;
    if (adds[e] != nullptr) {  // 0 + addend
      if (adds[e] != ptrs[e][2] &&
          hipMemcpyAsync(const_cast<void*>(ptrs[e][2]), adds[e], static_cast<size_t>(m) * n * 2, hipMemcpyDeviceToDevice, s) != hipSuccess)
        return fail(WX_ERR_LAUNCH, "wx_dual_gemm_add: copy of the addend failed");
      gemm_path_note(WX_GEMM_PATH_ADD_COPY);
      p.g[e].m = 0;
      continue;
    }
    const int64_t n16 = m * n / 8;  // n is a multiple of 8 and the buffer 16-byte aligned
    const int64_t want = (n16 + 255) / 256, cap = static_cast<int64_t>(device_cu_count()) * 8;
    hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>(want < cap ? want : cap)), dim3(256), 0, s,
                       static_cast<u32x4*>(const_cast<void*>(ptrs[e][2])), n16);
    if (int rc = check_launch("zero_fill_kernel")) return rc;
    gemm_path_note(WX_GEMM_PATH_ZERO_FILL);
    p.g[e].m = 0;
  }
  if ((p.g[0].m == 0 || n0 == 0) && (p.g[1].m == 0 || n1 == 0)) return WX_OK;
  const int64_t mm0 = p.g[0].m, mm1 = p.g[1].m;  // row counts left after the empty contractions are done
  // K-major operands (A stored [k, m], B stored [k, n]) advance by whole rows of K through a 32-bit byte count
  bool fits = true;
  for (int e = 0; e < 2; ++e) {
    if (trans_a && dims[e][2] * dims[e][0] * 2 >= (1ll << 32)) fits = false;
    if (!trans_b && dims[e][2] * dims[e][1] * 2 >= (1ll << 32)) fits = false;
  }
  if (fits) {
    const int64_t tiles = ceil_div(mm0, BigTile::BM) * ceil_div(n0, BigTile::BN) + ceil_div(mm1, BigTile::BM) * ceil_div(n1, BigTile::BN);
    const char* who = "dual_gemm_kernel<generic>";
    gemm_path_note(WX_GEMM_PATH_MFMA);
    // (the host knows both problems' sizes: it settles the tile shape and the split of a ragged last round itself)
    const int64_t by_expert[2] = {ceil_div(mm0, BigTile::BM) * ceil_div(n0, BigTile::BN),
                                  ceil_div(mm1, BigTile::BM) * ceil_div(n1, BigTile::BN)};
    if (!trans_a && trans_b) return launch_mfma<kGeneric, false, false>(p, tiles, tiles, s, who, by_expert);
    if (!trans_a && !trans_b) return launch_mfma<kGeneric, false, true>(p, tiles, tiles, s, who, by_expert);
    if (trans_a && trans_b) return launch_mfma<kGeneric, true, false>(p, tiles, tiles, s, who, by_expert);
    return launch_mfma<kGeneric, true, true>(p, tiles, tiles, s, who, by_expert);
  }
  gemm_path_note(WX_GEMM_PATH_FMA);
  hipLaunchKernelGGL(dual_gemm_reference_layout_kernel, dim3(device_cu_count() * 4), dim3(256), 0, s, p, trans_a, trans_b);
  return check_launch("dual_gemm_reference_layout_kernel");
}
}  // namespace

extern "C" int wx_qkv_rope_proj(const void* x, const void* weight, const void* bias, const uint32_t* rope_table,
                                int table_width, void* out, int64_t num_tokens, int64_t hidden, int n_q_heads,
                                int n_kv_heads, int head_dim, wx_stream_t stream) {
  const char* who = "wx_qkv_rope_proj";
  if (n_q_heads < 0 || n_kv_heads < 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: negative head count", who);
  if (head_dim != 128)
    return fail(WX_ERR_UNSUPPORTED, "%s: head_dim %d; the epilogue rotates heads of 128 channels", who, head_dim);
  if (table_width != head_dim / 2 && table_width != head_dim)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: table_width %d must be %d (channels d and d + %d share an entry) or %d", who,
                table_width, head_dim / 2, head_dim / 2, head_dim);
  const int64_t n = static_cast<int64_t>(n_q_heads + 2 * n_kv_heads) * head_dim;
  if (int rc = check_dims(who, num_tokens, n, hidden)) return rc;
  if (num_tokens == 0 || n == 0) return WX_OK;
  if (hidden == 0) return fail(WX_ERR_UNSUPPORTED, "%s: hidden must be positive", who);
  if (!x || !weight || !out || !rope_table) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  if ((reinterpret_cast<uintptr_t>(bias) & 1) || (reinterpret_cast<uintptr_t>(rope_table) & 3))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: misaligned bias or table", who);
  Params p{};
  Group& g = p.g[0];
  g.a = static_cast<const __bf16*>(x);
  g.b0 = static_cast<const __bf16*>(weight);
  g.c = static_cast<__bf16*>(out);
  g.m = static_cast<int>(num_tokens); g.n = static_cast<int>(n); g.k = static_cast<int>(hidden);
  g.lda = g.ldb = static_cast<int>(hidden);
  g.ldc = static_cast<int>(n);
  p.bias = static_cast<const __bf16*>(bias);
  p.rope_table = rope_table;
  p.rope_cols = (n_q_heads + n_kv_heads) * head_dim;
  p.rope_width = table_width;
  // Tiles whose wavefronts cover whole heads only (a 64-column wave tile would split a rotation pair): the large
  // tile, and for a ragged last round (see tail_split_point) a second launch of 128 x 128 tiles with 32 x 128 wave tiles
  using Tile = BigTileFor<kQkvRope>;
  using Tail = TailTileFor<kQkvRope>;
  const int cus = device_cu_count();
  const int64_t tiles = ceil_div(num_tokens, Tile::BM) * ceil_div(n, Tile::BN);
  const bool split = tiles < INT32_MAX && tail_split_point(static_cast<int>(tiles), 0, g.k, 0, cus) != tiles;
  p.split = split ? 1 : 0;
  p.split_cus = cus;
  hipStream_t s = as_stream(stream);
  if (table_width == head_dim) {
    hipLaunchKernelGGL((dual_gemm_kernel<kQkvRopeFull, Tile, false, false>), dim3(cus), dim3(Tile::kThreads), 0, s, p);
    if (split) {
      p.split = 2;
      hipLaunchKernelGGL((dual_gemm_kernel<kQkvRopeFull, Tail, false, false>), dim3(cus * Tail::kWgPerCu),
                         dim3(Tail::kThreads), 0, s, p);
    }
  } else {
    hipLaunchKernelGGL((dual_gemm_kernel<kQkvRope, Tile, false, false>), dim3(cus), dim3(Tile::kThreads), 0, s, p);
    if (split) {
      p.split = 2;
      hipLaunchKernelGGL((dual_gemm_kernel<kQkvRope, Tail, false, false>), dim3(cus * Tail::kWgPerCu),
                         dim3(Tail::kThreads), 0, s, p);
    }
  }
  return check_launch("dual_gemm_kernel<qkv_rope>");
}

extern "C" size_t wx_tiled_bytes(int64_t rows, int64_t cols) {
  if (rows < 0 || cols < 0) return 0;
  return static_cast<size_t>(tiled_bytes(rows, (cols + kBlkCols - 1) / kBlkCols * kBlkCols));
}

extern "C" int64_t wx_padded_sorted_rows(int64_t rows) { return rows < 0 ? 0 : padded_sorted_rows(rows); }

extern "C" int wx_pack_tiled(const void* src, void* dst, int64_t rows, int64_t cols, wx_stream_t stream) {
  if (rows < 0 || cols < 0) return fail(WX_ERR_INVALID_ARGUMENT, "wx_pack_tiled: negative size");
  if (cols % kBlkCols != 0)
    return fail(WX_ERR_UNSUPPORTED, "wx_pack_tiled: cols (%lld) must be a multiple of 32", static_cast<long long>(cols));
  if (rows == 0 || cols == 0) return WX_OK;
  if (!src || !dst) return fail(WX_ERR_INVALID_ARGUMENT, "wx_pack_tiled: null pointer");
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "wx_pack_tiled: buffers must be 16-byte aligned");
  const int64_t chunks = tiled_row_blocks(rows) * kBlkRows * (cols / 8);
  const int64_t want = (chunks + 255) / 256;
  const int64_t cap = static_cast<int64_t>(device_cu_count()) * 16;
  hipLaunchKernelGGL(pack_tiled_kernel, dim3(static_cast<unsigned>(want < cap ? want : cap)), dim3(256), 0,
                     as_stream(stream), static_cast<const u32x4*>(src), static_cast<unsigned char*>(dst), rows, cols);
  return check_launch("pack_tiled_kernel");
}

namespace {

struct FfnArgs {
  const void *x, *gate[2], *up[2], *down[2];
  void *out, *hmid;
  const int64_t* host_rows;  // optional: rows of each expert as the caller knows them on the host
  const int32_t* offsets;
  int64_t rows, hidden, inter[2];
  const int32_t* out_row_id = nullptr;  // optional: sorted row r of the result goes to row out_row_id[r] of `out`
  void *keep_gate = nullptr, *keep_up = nullptr;  // optional: the gate / up projections, K-tiled like hmid
  const void* residual = nullptr;  // optional (with out_row_id): rows added to the result, laid out like `out`
  const void* x_rows = nullptr;    // optional: the activations in token order; `x` is then built by the fused launch
};

int check_ffn(const char* who, const FfnArgs& a, bool need_gate_up, bool need_down) {
  if (int rc = check_dims(who, a.rows, a.inter[0], a.hidden)) return rc;
  if (int rc = check_dims(who, a.rows, a.hidden, a.inter[1])) return rc;
  if (a.hidden % kBlkCols != 0 || a.inter[0] % kBlkCols != 0 || a.inter[1] % kBlkCols != 0)
    return fail(WX_ERR_UNSUPPORTED, "%s: hidden and intermediate sizes must be multiples of 32", who);
  if (a.host_rows != nullptr && (a.host_rows[0] < 0 || a.host_rows[1] < 0 || a.host_rows[0] + a.host_rows[1] != a.rows))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: host_rows_per_expert must be non-negative and sum to num_rows", who);
  if (a.hidden == 0 || a.inter[0] == 0 || a.inter[1] == 0)
    return fail(WX_ERR_UNSUPPORTED, "%s: hidden and both intermediate sizes must be positive", who);
  if (a.rows == 0) return WX_OK;
  if (!a.offsets || !a.hmid || (need_gate_up && !a.x) || (need_down && !a.out))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  for (int e = 0; e < 2; ++e) {
    if (a.inter[e] == 0) continue;
    if ((need_gate_up && (!a.gate[e] || !a.up[e])) || (need_down && !a.down[e]))
      return fail(WX_ERR_INVALID_ARGUMENT, "%s: null weight pointer for expert %d", who, e);
  }
  const int64_t max_inter = a.inter[0] > a.inter[1] ? a.inter[0] : a.inter[1];
  if (padded_sorted_rows(a.rows) * max_inter * 2 >= (1ll << 40))
    return fail(WX_ERR_UNSUPPORTED, "%s: intermediate too large", who);
  return WX_OK;
}

// hmid_e = silu(x_e @ gate_e^T) * (x_e @ up_e^T), K-tiled per expert
Params gate_up_params(const FfnArgs& a) {
  Params p{};
  for (int e = 0; e < 2; ++e) {
    Group& g = p.g[e];
    g.a = static_cast<const __bf16*>(a.x);
    g.b0 = static_cast<const __bf16*>(a.gate[e]);
    g.b1 = static_cast<const __bf16*>(a.up[e]);
    g.c = static_cast<__bf16*>(a.hmid);
    g.m = 0; g.n = static_cast<int>(a.inter[e]); g.k = static_cast<int>(a.hidden);
    g.lda = static_cast<int>(padded_sorted_rows(a.rows) / kBlkRows);  // row blocks of the tiled activations
    g.ldb = static_cast<int>(tiled_row_blocks(a.inter[e]));           // row blocks of the tiled weights
    g.ldc = 0;                                                        // set on the device from the row counts
    g.a_row0 = 0;
  }
  p.offsets = a.offsets;
  p.keep_gate = static_cast<__bf16*>(a.keep_gate);
  p.keep_up = static_cast<__bf16*>(a.keep_up);
  return p;
}

int launch_gate_up(const FfnArgs& a, hipStream_t s) {
  const Params p = gate_up_params(a);
  const int64_t t0 = ceil_div(a.inter[0], BigTile::BN / 2), t1 = ceil_div(a.inter[1], BigTile::BN / 2);
  if (a.host_rows != nullptr) {  // the caller knows the split: one launch of the right tile shape
    const int64_t by_expert[2] = {ceil_div(a.host_rows[0], BigTile::BM) * t0, ceil_div(a.host_rows[1], BigTile::BM) * t1};
    const int64_t tiles = by_expert[0] + by_expert[1];
    return launch_mfma<kGateUp>(p, tiles, tiles, s, "dual_gemm_kernel<gate_up>", by_expert);
  }
  // the split of the rows between the experts is only known on the device: bound the tile count from the total
  const int64_t row_tiles = ceil_div(a.rows, BigTile::BM);
  return launch_mfma<kGateUp>(p, row_tiles * (t0 < t1 ? t0 : t1), (row_tiles + 1) * (t0 > t1 ? t0 : t1), s,
                              "dual_gemm_kernel<gate_up>");
}

// out_e = hmid_e @ down_e^T, row-major, expert e's rows start at offsets[e]
Params down_params(const FfnArgs& a) {
  Params p{};
  for (int e = 0; e < 2; ++e) {
    Group& g = p.g[e];
    g.a = static_cast<const __bf16*>(a.hmid);
    g.b0 = static_cast<const __bf16*>(a.down[e]);
    g.b1 = nullptr;
    g.c = static_cast<__bf16*>(a.out);
    g.m = 0; g.n = static_cast<int>(a.hidden); g.k = static_cast<int>(a.inter[e]);
    g.lda = 0;  // set on the device from the row counts
    g.ldb = static_cast<int>(tiled_row_blocks(a.hidden));
    g.ldc = static_cast<int>(a.hidden);
    g.a_row0 = 0;
  }
  p.offsets = a.offsets;
  p.scatter = a.out_row_id;
  p.residual = static_cast<const __bf16*>(a.residual);
  return p;
}

int launch_down(const FfnArgs& a, hipStream_t s) {
  const Params p = down_params(a);
  const int64_t col_tiles = ceil_div(a.hidden, BigTile::BN);
  if (a.host_rows != nullptr) {
    const int64_t by_expert[2] = {ceil_div(a.host_rows[0], BigTile::BM) * col_tiles, ceil_div(a.host_rows[1], BigTile::BM) * col_tiles};
    const int64_t tiles = by_expert[0] + by_expert[1];
    return launch_mfma<kDown>(p, tiles, tiles, s, "dual_gemm_kernel<down>", by_expert);
  }
  const int64_t row_tiles = ceil_div(a.rows, BigTile::BM);
  return launch_mfma<kDown>(p, row_tiles * col_tiles, (row_tiles + 1) * col_tiles, s, "dual_gemm_kernel<down>");
}

// Both launches as one (ffn_fused_kernel), for the shapes where each is a single round of small tiles with the row
// counts known on the host -- a denoise step.  With a.x_rows the gate/up tiles read the token rows themselves (the
// permute happens in their loads; a.x is not touched).  Returns 1 when the shape is not of that kind (nothing launched).
// Whether the one launch that last used workspace `ws` from this thread ran on the same weights (they are then
// taken to be in the caches still, and the launch does not pull them in ahead of its K loops: in a loop over one
// layer that would cost 0.9 us per launch, where for a model's layers, each with weights of its own, it saves 2).
// A guess that only decides this; a few workspaces (streams) per thread are remembered.
bool weights_of_last_launch(const void* ws, const FfnArgs& a) {
  struct Seen { const void* ws; const void* w[6]; };
  constexpr int kSeen = 8;
  thread_local Seen seen[kSeen] = {};
  thread_local int next = 0;
  const void* w[6] = {a.gate[0], a.up[0], a.down[0], a.gate[1], a.up[1], a.down[1]};
  for (Seen& s : seen) {
    if (s.ws != ws) continue;
    bool same = true;
    for (int i = 0; i < 6; ++i) { same = same && s.w[i] == w[i]; s.w[i] = w[i]; }
    return same;
  }
  Seen& s = seen[next];
  next = (next + 1) % kSeen;
  s.ws = ws;
  for (int i = 0; i < 6; ++i) s.w[i] = w[i];
  return false;
}

constexpr size_t kFusedWorkspaceInts = 2 * static_cast<size_t>(kFusedCounters) + 1;  // two counter arrays, then the error flag
int launch_ffn_fused(const FfnArgs& a, int* ws, hipStream_t s) {
  if (ws == nullptr || a.keep_gate != nullptr) return 1;
  // (whatever the real split of the rows: the counters hold this many row blocks per expert)
  if (a.rows > static_cast<int64_t>(kFusedMaxRowBlocks) * SmallTile::BM) return 1;
  // (token rows are addressed with 31-bit byte offsets)
  if (a.x_rows != nullptr && (a.out_row_id == nullptr || a.rows * a.hidden * 2 >= (1ll << 31))) return 1;
  const int cus = device_cu_count();
  int64_t gate_tiles = 0, down_tiles = 0;
  int need[2] = {0, 0};
  const int64_t down_cols = ceil_div(a.hidden, SmallTile::BN);
  for (int e = 0; e < 2; ++e) {
    need[e] = static_cast<int>(ceil_div(a.inter[e], SmallTile::BN / 2));
    if (a.host_rows != nullptr) {
      const int64_t row_blocks = ceil_div(a.host_rows[e], SmallTile::BM);
      gate_tiles += row_blocks * need[e];
      down_tiles += row_blocks * down_cols;
    }
  }
  const bool rows_known = a.host_rows != nullptr;
  if (!rows_known) {
    // The split of the rows is only known on the device.  The launch is right for any split (workgroups take as
    // many tiles as there are), so what the host has to settle is whether it is the faster form whatever the split.
    // Up to two rows per CU it is: 24-27 against 29-34 us with every row on the narrow expert, 2-9 % ahead with a
    // mix, within 4 % with every row on the wide expert (256 and 512 rows, experts 11008 / 1024).  Beyond that, rows
    // on the wide expert cost the one workgroup of producers per CU more than they cost the separate launches' large
    // tiles (+12 % at 1024 rows, +19 % at 2048, against -25 % / -31 % with none); with two workgroups of producers
    // per CU the consumers land wherever a producer has left, two of them on one CU while others idle (+25 % on a
    // half-and-half split of 1024 rows).  So larger problems take the one launch only with the host's row counts.
    if (a.rows > 2 * cus) return 1;
    gate_tiles = down_tiles = cus;
  }
  if (gate_tiles == 0 || gate_tiles > cus || down_tiles > cus) return 1;
  Params pg = gate_up_params(a), pd = down_params(a);
  pg.gate = pd.gate = 0;
  pg.split = pd.split = 0;
  FusedSync fs{};
  fs.ready = ws;
  fs.passed = ws + kFusedCounters;
  fs.error = ws + 2 * kFusedCounters;
  fs.need[0] = need[0];
  fs.need[1] = need[1];
  fs.consumers = static_cast<int>(down_cols);
  if (!weights_of_last_launch(ws, a)) {
    for (int e = 0; e < 2; ++e) {
      fs.warm_b[e][0] = pg.g[e].b0;
      fs.warm_b[e][1] = pg.g[e].b1;
      fs.warm_ldb[e] = pg.g[e].ldb;
    }
    fs.warm_k = static_cast<int>(a.hidden);
  }
  fs.x = static_cast<const __bf16*>(a.x_rows);
  fs.gather = a.out_row_id;
  const int producers = static_cast<int>((gate_tiles + kXcds - 1) / kXcds * kXcds);
  const int consumers = static_cast<int>((down_tiles + kXcds - 1) / kXcds * kXcds);
  if (a.x_rows != nullptr)
    hipLaunchKernelGGL(ffn_fused_kernel<true>, dim3(producers + consumers), dim3(SmallTile::kThreads), 0, s, pg, pd, fs, producers);
  else
    hipLaunchKernelGGL(ffn_fused_kernel<false>, dim3(producers + consumers), dim3(SmallTile::kThreads), 0, s, pg, pd, fs, producers);
  return check_launch("ffn_fused_kernel");
}

}  // namespace

extern "C" size_t wx_ffn_fused_workspace_bytes(void) { return kFusedWorkspaceInts * sizeof(int); }

extern "C" int wx_dual_swiglu_ffn_fused(const void* x_rows, void* x_tiled, void* out, const void* residual,
                                        const int32_t* expert_offsets, const void* gate0, const void* up0,
                                        const void* down0, const void* gate1, const void* up1, const void* down1,
                                        void* hmid, int64_t num_rows, int64_t hidden, int64_t inter0, int64_t inter1,
                                        const int64_t* host_rows_per_expert, const int32_t* out_row_id,
                                        void* workspace, wx_stream_t stream) {
  const char* who = "wx_dual_swiglu_ffn_fused";
  FfnArgs a{x_tiled, {gate0, gate1}, {up0, up1}, {down0, down1}, out, hmid, host_rows_per_expert, expert_offsets,
            num_rows, hidden, {inter0, inter1}, out_row_id};
  if (int rc = check_ffn(who, a, true, true)) return rc;
  if (num_rows == 0) return WX_OK;
  if (residual != nullptr) {
    if (!out_row_id) return fail(WX_ERR_INVALID_ARGUMENT, "%s: a residual needs out_row_id (the sum is formed in token order)", who);
    if (reinterpret_cast<uintptr_t>(residual) & 15) return fail(WX_ERR_INVALID_ARGUMENT, "%s: residual must be 16-byte aligned", who);
    a.residual = residual;
  }
  if (x_rows != nullptr) {
    if (!out_row_id) return fail(WX_ERR_INVALID_ARGUMENT, "%s: x_rows needs out_row_id (the rows are gathered through it)", who);
    if (reinterpret_cast<uintptr_t>(x_rows) & 15) return fail(WX_ERR_INVALID_ARGUMENT, "%s: x_rows must be 16-byte aligned", who);
    a.x_rows = x_rows;
  }
  if (reinterpret_cast<uintptr_t>(workspace) & 3) return fail(WX_ERR_INVALID_ARGUMENT, "%s: workspace must be 4-byte aligned", who);
  const int rc = launch_ffn_fused(a, static_cast<int*>(workspace), as_stream(stream));
  if (rc <= 0) return rc;
  if (x_rows != nullptr)
    if (int rc2 = wx_permute_rows_tiled(x_rows, x_tiled, nullptr, out_row_id, expert_offsets, num_rows, hidden, stream)) return rc2;
  if (int rc2 = launch_gate_up(a, as_stream(stream))) return rc2;
  return launch_down(a, as_stream(stream));
}

extern "C" int wx_dual_swiglu_gate_up(const void* x_tiled, void* hmid, const int32_t* expert_offsets,
                                      const void* gate0, const void* up0, const void* gate1, const void* up1,
                                      int64_t num_rows, int64_t hidden, int64_t inter0, int64_t inter1,
                                      const int64_t* host_rows_per_expert, wx_stream_t stream) {
  const FfnArgs a{x_tiled, {gate0, gate1}, {up0, up1}, {nullptr, nullptr}, nullptr, hmid, host_rows_per_expert, expert_offsets,
                  num_rows, hidden, {inter0, inter1}};
  if (int rc = check_ffn("wx_dual_swiglu_gate_up", a, true, false)) return rc;
  if (num_rows == 0) return WX_OK;
  return launch_gate_up(a, as_stream(stream));
}

extern "C" int wx_dual_swiglu_gate_up_keep(const void* x_tiled, void* hmid, void* gate_keep, void* up_keep,
                                           const int32_t* expert_offsets, const void* gate0, const void* up0,
                                           const void* gate1, const void* up1, int64_t num_rows, int64_t hidden,
                                           int64_t inter0, int64_t inter1, const int64_t* host_rows_per_expert,
                                           wx_stream_t stream) {
  FfnArgs a{x_tiled, {gate0, gate1}, {up0, up1}, {nullptr, nullptr}, nullptr, hmid, host_rows_per_expert, expert_offsets,
            num_rows, hidden, {inter0, inter1}};
  if (int rc = check_ffn("wx_dual_swiglu_gate_up_keep", a, true, false)) return rc;
  if (num_rows == 0) return WX_OK;
  if (!gate_keep || !up_keep) return fail(WX_ERR_INVALID_ARGUMENT, "wx_dual_swiglu_gate_up_keep: null pointer");
  if ((reinterpret_cast<uintptr_t>(gate_keep) | reinterpret_cast<uintptr_t>(up_keep)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "wx_dual_swiglu_gate_up_keep: buffers must be 16-byte aligned");
  a.keep_gate = gate_keep;
  a.keep_up = up_keep;
  return launch_gate_up(a, as_stream(stream));
}

extern "C" int wx_dual_down_proj(const void* hmid, void* out, const int32_t* expert_offsets, const void* down0,
                                 const void* down1, int64_t num_rows, int64_t hidden, int64_t inter0,
                                 int64_t inter1, const int64_t* host_rows_per_expert, const int32_t* out_row_id,
                                 wx_stream_t stream) {
  const FfnArgs a{nullptr, {nullptr, nullptr}, {nullptr, nullptr}, {down0, down1}, out, const_cast<void*>(hmid),
                  host_rows_per_expert, expert_offsets, num_rows, hidden, {inter0, inter1}, out_row_id};
  if (int rc = check_ffn("wx_dual_down_proj", a, false, true)) return rc;
  if (num_rows == 0) return WX_OK;
  return launch_down(a, as_stream(stream));
}

extern "C" int wx_dual_down_proj_residual(const void* hmid, void* out, const void* residual,
                                          const int32_t* expert_offsets, const void* down0, const void* down1,
                                          int64_t num_rows, int64_t hidden, int64_t inter0, int64_t inter1,
                                          const int64_t* host_rows_per_expert, const int32_t* out_row_id,
                                          wx_stream_t stream) {
  const char* who = "wx_dual_down_proj_residual";
  FfnArgs a{nullptr, {nullptr, nullptr}, {nullptr, nullptr}, {down0, down1}, out, const_cast<void*>(hmid),
            host_rows_per_expert, expert_offsets, num_rows, hidden, {inter0, inter1}, out_row_id};
  if (int rc = check_ffn(who, a, false, true)) return rc;
  if (num_rows == 0) return WX_OK;
  if (!residual || !out_row_id)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: residual and out_row_id are required (the sum is formed in token order)", who);
  if (reinterpret_cast<uintptr_t>(residual) & 15) return fail(WX_ERR_INVALID_ARGUMENT, "%s: residual must be 16-byte aligned", who);
  a.residual = residual;
  return launch_down(a, as_stream(stream));
}

extern "C" int wx_dual_swiglu_ffn(const void* x_tiled, void* out, const int32_t* expert_offsets, const void* gate0,
                                  const void* up0, const void* down0, const void* gate1, const void* up1,
                                  const void* down1, void* hmid, int64_t num_rows, int64_t hidden, int64_t inter0,
                                  int64_t inter1, const int64_t* host_rows_per_expert, const int32_t* out_row_id,
                                  wx_stream_t stream) {
  const FfnArgs a{x_tiled, {gate0, gate1}, {up0, up1}, {down0, down1}, out, hmid, host_rows_per_expert, expert_offsets,
                  num_rows, hidden, {inter0, inter1}, out_row_id};
  if (int rc = check_ffn("wx_dual_swiglu_ffn", a, true, true)) return rc;
  if (num_rows == 0) return WX_OK;
  if (int rc = launch_gate_up(a, as_stream(stream))) return rc;
  return launch_down(a, as_stream(stream));
}
