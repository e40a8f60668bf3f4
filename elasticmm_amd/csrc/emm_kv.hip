// libemm_kv — KV-cache data-movement kernels for gfx950 (MI355X) behind the C ABI
// declared in include/emm_kv.h.
//
// Everything here is HBM-bandwidth work. The shape every kernel follows was found
// by measurement on MI355X: a 256-thread workgroup moves one 4 KiB tile, each lane
// issues ONE 16-byte non-temporal load and ONE 16-byte store, every wave
// instruction covers 1 KiB of contiguous memory, and stores are system-scope
// write-through (sc0 sc1). Unrolled or persistent variants are slower on this part
// (the memory counter of gfx9 retires loads and stores in order, so a lane that
// loads after it has stored waits for a write acknowledgement). Block-table and
// slot-mapping entries are wave-uniform: they are fetched once per wave and all
// address arithmetic that depends on them stays in scalar registers; loads that do
// not depend on them are issued before they are waited for.
//
// Pool layout (per layer): [num_kv, num_blocks, chunk] contiguous, where
// chunk = block_size * num_kv_heads * head_dim elements.
// Transfer-buffer layout: [num_layers, num_kv, n, chunk] contiguous.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <string.h>
#include <type_traits>

#include "emm_kv.h"

namespace {

// ----------------------------------------------------------------------------
// error reporting
// ----------------------------------------------------------------------------
thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return fail(EMM_ELAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return EMM_OK;
}

// ----------------------------------------------------------------------------
// vector types and streaming accessors
// ----------------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Cache policies of the streaming accessors. Loads are always non-temporal.
//   0  store nt                (compiler builtin)
//   1  store sc0 sc1           (system-scope write-through)
//   2  store sc0 sc1 nt
//   3  plain load / plain store
// (the block-move kernels instantiate 0 and 1; 2 and 3 exist for experiments)
// The sc0/sc1 forms exist only as instruction modifiers, so 16-byte stores under
// policies 1 and 2 are emitted with a one-line asm statement (a vector store).
// Every pointer these kernels dereference is device (global) memory. Saying so in
// the pointer type keeps the accesses global_load / global_store even where a
// pointer has passed through an opaque asm statement (a generic pointer would
// become a slower flat access).
#define EMM_GLOBAL __attribute__((address_space(1)))

template <typename V, bool NT>
__device__ __forceinline__ V ld(const char *p) {
  const EMM_GLOBAL V *g = (const EMM_GLOBAL V *)(p);
  if constexpr (NT)
    return __builtin_nontemporal_load(g);
  else
    return *g;
}

template <typename V, bool NT>
__device__ __forceinline__ void st(char *p, V v) {
  EMM_GLOBAL V *g = (EMM_GLOBAL V *)(p);
  if constexpr (NT)
    __builtin_nontemporal_store(v, g);
  else
    *g = v;
}

template <typename V, int POLICY>
__device__ __forceinline__ V ld_stream(const char *p) {
  return ld<V, POLICY != 3>(p);
}

template <typename V, int POLICY>
__device__ __forceinline__ void st_stream(char *p, V v) {
  // A store of more than 8 bytes reads its data registers after it has issued; the
  // next instruction must not overwrite them. The compiler inserts that wait state
  // for its own stores but cannot see inside an asm statement, hence the s_nop.
  if constexpr (sizeof(V) == 8 && (POLICY == 1 || POLICY == 2)) {
    asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
  } else if constexpr (sizeof(V) == 16 && POLICY == 1) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
  } else if constexpr (sizeof(V) == 16 && POLICY == 2) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
  } else {
    st<V, POLICY != 3>(p, v);
  }
}

constexpr int kThreads = 256; // 4 wavefronts of 64 lanes (append / dequant / concat kernels)

// A tile is U * T vectors; lane `tid` owns vectors (u * T + tid). All U loads of a
// tile are in flight before the first store. `limit` is the number of bytes valid
// from the tile start on (tail tiles are predicated per lane): lanes past the end
// re-read vector 0 (always valid, limit > 0) so the loads stay unconditional;
// only the stores are predicated.
template <typename V, int T, int U, int POLICY>
__device__ __forceinline__ void load_tile(V (&v)[U], const char *__restrict__ src, int64_t limit) {
  constexpr int64_t VB = sizeof(V);
  const int64_t lane_off = (int64_t)threadIdx.x * VB;
  if (limit >= (int64_t)U * T * VB) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      v[u] = ld_stream<V, POLICY>(src + lane_off + (int64_t)u * T * VB);
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t off = lane_off + (int64_t)u * T * VB;
      v[u] = ld_stream<V, POLICY>(src + (off < limit ? off : 0));
    }
  }
}

template <typename V, int T, int U, int POLICY>
__device__ __forceinline__ void store_tile(const V (&v)[U], char *__restrict__ dst, int64_t limit) {
  constexpr int64_t VB = sizeof(V);
  const int64_t lane_off = (int64_t)threadIdx.x * VB;
  if (limit >= (int64_t)U * T * VB) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      st_stream<V, POLICY>(dst + lane_off + (int64_t)u * T * VB, v[u]);
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t off = lane_off + (int64_t)u * T * VB;
      if (off < limit) st_stream<V, POLICY>(dst + off, v[u]);
    }
  }
}

template <typename V, int T, int U, int POLICY>
__device__ __forceinline__ void copy_tile(const char *__restrict__ src, char *__restrict__ dst,
                                          int64_t limit) {
  V v[U];
  load_tile<V, T, U, POLICY>(v, src, limit);
  store_tile<V, T, U, POLICY>(v, dst, limit);
}

// ----------------------------------------------------------------------------
// block move: pack / unpack / copy_blocks / migrate
// ----------------------------------------------------------------------------
// One side of a move is either a block pool (one base pointer per (layer, K|V)
// plane, block chosen through an int64 index array) or a linear transfer
// buffer [planes, n, chunk].
//
// What bounds these kernels is not instruction issue but the length of the chain of
// dependent memory round trips a wave goes through before its data load is in flight
// (measured: with the pool side read at random the memory system is not saturated — its
// queues report 15x fewer stalls for lack of DRAM credits than for a sequential copy —
// so every round trip a wave waits for shows up as lost throughput). The chain is kept
// at its minimum of two:
//   1. block id (scalar load through the index pointer) and plane base (scalar load from
//      the table in the argument block), issued together and waited for once;
//   2. the data.
// To that end the scalar arguments are explicit kernel parameters in the order in which
// they are needed, so that the hardware preloads them into scalar registers before the
// wave starts (kernarg preload, -mllvm -amdgpu-kernarg-preload-count): no round trip is
// spent on fetching them. Loads from a linear source depend on no id and are issued
// before that single wait. Launch-order variants and tail handling are template
// parameters, so the common path carries no branch and no extra argument.
constexpr int kMaxPlanes = 2 * EMM_MAX_LAYERS;
constexpr int kMaxGridY = 65535;
constexpr int kRun = 16; // blocks per plane visit in the pool-to-pool order

struct PlaneTable {
  char *base[kMaxPlanes]; // base of each (layer, kv) plane
};
template <int N>
struct PlaneTables {
  PlaneTable t[N]; // pack: source; unpack: destination; pool-to-pool: source, destination
};

// Block ids carried in the argument block itself (host-side tables of up to EMM_MAX_INLINE_IDS
// entries): no device-side table, no host-to-device copy, and the id fetch is a scalar load from the
// argument block, which every workgroup of the launch shares. 0xFFFFFFFF marks an id to skip.
struct InlineIds {
  uint32_t id[EMM_MAX_INLINE_IDS];
};
struct NoIds {};

constexpr int kPack = 0, kUnpack = 1, kPoolToPool = 2;
// Launch orders (grid x is always the tile inside a chunk):
//  plain    y = block, z = plane: walks the transfer buffer linearly.
//  grouped  y = plane * 2^g + position, z = group: groups of 2^g blocks per plane visit. Used for
//           long scatters: visiting a plane for thousands of blocks in a row keeps all writes inside
//           that plane's address window, which this memory system serves about 12 % slower than
//           writes spread over the whole pool.
//  runs     y = plane * kRun + position in a run of kRun consecutive blocks, z = run, every plane
//           starting at its own run: the workgroups in flight at any moment touch every plane of
//           the pool, while a table of consecutive ids still gives sequential runs. Used when both
//           sides are pools (about 12 % faster there; slower with a linear side, which would be
//           read as one stream per plane).
constexpr int kOrderPlain = 0, kOrderGrouped = 1, kOrderRuns = 2;
// Tile -> XCD mappings, flags in the top bits of `order_arg`. Workgroups go to the 8 XCDs round-robin in dispatch
// order (x fastest), so with the plain mapping every XCD takes every eighth 4 KiB tile and the tiles of a 16 KiB
// chunk land on 4 XCDs. Inside every window of 8 chunks (8 * tiles-per-chunk consecutive workgroups):
//   kXcdPairs  the workgroups q and q + 8 of every 16 take two neighbouring tiles: every XCD requests 8 KiB
//              contiguous (tiles per chunk must be even);
//   kXcdChunk  workgroup q takes tile q / 8 of chunk q % 8: every XCD requests whole chunks.
// Both are bijections on the window's (x, y); what is left of y past the last whole window keeps the plain
// mapping. The host decides per launch (xcd_mapping below).
constexpr uint32_t kXcdChunk = 0x80000000u, kXcdPairs = 0x40000000u, kXcdMask = kXcdChunk | kXcdPairs;

// (bx, by) of the tile this workgroup moves. `whole` = the y covered by whole windows of 8.
__device__ __forceinline__ void xcd_map(uint32_t mode, uint32_t tpc, uint32_t whole, uint32_t &bx, uint32_t &by) {
  if (!(mode & kXcdMask) || by >= whole) return;
  const uint32_t lin = bx + tpc * (by & 7u); // position in the window
  if (mode & kXcdChunk) {
    by = (by & ~7u) | (lin & 7u);
    bx = lin >> 3;
  } else {
    const uint32_t t = (lin & ~15u) + 2u * (lin & 7u) + ((lin >> 3) & 1u); // 8 * tpc is a multiple of 16
    const uint32_t c = (tpc & (tpc - 1u)) == 0u ? t >> __builtin_ctz(tpc) : t / tpc;
    by = (by & ~7u) + c;
    bx = t - c * tpc;
  }
}

// idx_a / idx_b: source / destination ids (PAIRS: idx_a holds (src, dst) pairs, idx_b unused).
// `n` = blocks of this launch (ids and linear buffer already offset to its first block),
// `order_arg` = log2 of the group size (grouped) or the per-plane rotation of the runs (runs).
// INLINE: the ids come from `ids` in the argument block (pack / unpack, plain order) instead.
template <typename V, int U, int KIND, int ORDER, bool FULL, bool PAIRS, int POLICY, bool INLINE = false>
__global__ __launch_bounds__(kThreads) void emm_block_move_kernel(
    const int64_t *__restrict__ idx_a, const int64_t *__restrict__ idx_b, char *lin,
    int64_t lin_plane_stride, int64_t chunk, uint32_t src_nb, uint32_t dst_nb, uint32_t n,
    uint32_t order_arg, const PlaneTables<KIND == kPoolToPool ? 2 : 1> tables,
    const std::conditional_t<INLINE, InlineIds, NoIds> ids) {
  constexpr int64_t TILE = (int64_t)U * kThreads * sizeof(V);
  constexpr bool SRC_POOL = KIND != kUnpack, DST_POOL = KIND != kPack;
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  xcd_map(order_arg, (uint32_t)((chunk + TILE - 1) / TILE) /* = gridDim.x */,
          ORDER == kOrderPlain ? (n & ~7u) : ~7u /* grouped / runs: y is a multiple of 8 per plane */, bx, by);
  order_arg &= ~kXcdMask;
  uint32_t pl, j;
  if constexpr (ORDER == kOrderRuns) {
    pl = by / kRun;
    const uint32_t runs = (n + kRun - 1) / kRun;
    uint32_t run = blockIdx.z + pl * order_arg; // order_arg = runs / planes
    if (run >= runs) run -= runs;
    j = run * kRun + (by % kRun);
    if (j >= n) return;
  } else if constexpr (ORDER == kOrderGrouped) {
    pl = by >> order_arg;
    j = (blockIdx.z << order_arg) + (by & ((1u << order_arg) - 1u));
    if (j >= n) return;
  } else {
    pl = blockIdx.z;
    j = by;
  }
  // round trip 1: ids and plane bases, all issued before the one wait below
  int64_t sb = 0, db = 0;
  if constexpr (INLINE) {
    static_assert(!INLINE || (KIND != kPoolToPool && ORDER == kOrderPlain && !PAIRS), "inline ids: pack / unpack only");
    if constexpr (SRC_POOL) sb = ids.id[j];
    if constexpr (DST_POOL) db = ids.id[j];
  } else if constexpr (PAIRS) {
    sb = idx_a[2 * (uint64_t)j];
    db = idx_a[2 * (uint64_t)j + 1];
  } else {
    if constexpr (SRC_POOL) sb = idx_a[j];
    if constexpr (DST_POOL) db = idx_b[j];
  }
  const char *src_plane = nullptr;
  char *dst_plane = nullptr;
  if constexpr (SRC_POOL) src_plane = tables.t[0].base[pl];
  if constexpr (DST_POOL) dst_plane = tables.t[KIND == kPoolToPool ? 1 : 0].base[pl];

  const int64_t tile_off = (int64_t)bx * TILE;
  const int64_t limit = FULL ? TILE : chunk - tile_off;
  char *linp = nullptr;
  if constexpr (KIND != kPoolToPool) linp = lin + (int64_t)pl * lin_plane_stride + (int64_t)j * chunk + tile_off;
  V v[U];
  if constexpr (!SRC_POOL) load_tile<V, kThreads, U, POLICY>(v, linp, limit); // needs no id
  asm volatile("" : "+s"(sb), "+s"(db), "+s"(src_plane), "+s"(dst_plane) : : "memory");
  if constexpr (SRC_POOL) {
    if ((uint64_t)sb >= (uint64_t)src_nb) return; // padding (negative) / out of range: skipped
    load_tile<V, kThreads, U, POLICY>(v, src_plane + sb * chunk + tile_off, limit); // round trip 2
  }
  char *dst;
  if constexpr (DST_POOL) {
    if ((uint64_t)db >= (uint64_t)dst_nb) return;
    dst = dst_plane + db * chunk + tile_off;
  } else {
    dst = linp;
  }
  store_tile<V, kThreads, U, POLICY>(v, dst, limit);
}

// Plain device-to-device copy with the same tile shape (the yardstick of the block moves).
template <typename V, int U, int POLICY>
__global__ __launch_bounds__(kThreads) void emm_stream_copy_kernel(const char *__restrict__ src,
                                                                   char *__restrict__ dst, int64_t nbytes) {
  constexpr int64_t TILE = (int64_t)U * kThreads * sizeof(V);
  const int64_t off = (int64_t)blockIdx.x * TILE;
  copy_tile<V, kThreads, U, POLICY>(src + off, dst + off, nbytes - off);
}

#ifdef EMM_BENCH_HOOKS
// Benchmark builds only (libemm_kv_hooks.so): launch variants selectable at run time.
int g_move_variant = 0;
inline int move_variant() { return g_move_variant; }
#else
constexpr int move_variant() { return 0; }
#endif

bool aligned(const void *p, int a) { return ((uintptr_t)p & (uintptr_t)(a - 1)) == 0; }

struct MoveArgs {
  const int64_t *idx_a;
  const int64_t *idx_b;
  char *lin;
  int64_t lin_plane_stride;
  int64_t chunk;
  uint32_t src_nb, dst_nb;
};

// The tile -> XCD mapping of a launch (kXcdPairs, kXcdChunk or 0). Measured by alternating the mappings on the same
// pools in one process, tables of 32 .. 4096 random blocks, against the plain mapping:
//  * unpack: pairs +0.5 .. +1.6 % on the Qwen2-7B pool (16 KiB chunks, 983 MB planes), +0.7 .. +3.0 % on the 80-layer
//    fp8 pool (327 MB planes); two cells of -0.6 / -0.7 % on other shapes;
//  * both sides pools (migrate, copy_blocks): pairs +0.2 .. +1.3 % on the Qwen2-7B pool, +1.3 .. +2.9 % on the 80-layer
//    fp8 pool; from 32 KiB chunks on whole chunks do better (+2 .. +6.9 % against +1.2 .. +4.5 %); copy_blocks in a
//    200 GB pool +1.2 .. +1.5 % at 512 and 4096 pairs, -0.3 % at 54 500;
//  * pack: pairs gain while the table is short against the plane it indexes and lose when it is not: Qwen2-7B pool
//    +1.0 / +2.1 / +2.3 / +1.6 / +0.7 % at 128 / 256 / 512 / 1000 / 2048 blocks, 80-layer fp8 pool +1.3 / -0.6 / -1.5 /
//    -1.6 / -2.2 %. The transfer-buffer side of a pack is a sequential stream, which wants the XCDs side by side on
//    4 KiB pieces (a plain copy loses 3 % with 8 KiB per XCD and 9 % with 16 KiB); the sparser the gather, the more
//    its side counts. Pairs are used up to blocks * 2 MiB = 1.25 x the plane's bytes. Whole chunks lose up to 8 %.
//  * the dequantising unpack keeps the plain mapping (pairs: 0 .. -0.4 % on the 80-layer pool).
// Launches of fewer than 96 blocks are left alone (their time is the launch ramp). The translation counters (UTCL1
// misses, UTCL2 busy) read the same with every mapping: the gain is not fewer page-table fetches; what changes is
// what each XCD requests at a time. Benchmark builds can force plain (bit 25), whole chunks (26) or pairs (27).
constexpr int kMapPack = 0, kMapUnpack = 1, kMapPoolToPool = 2, kMapDequant = 3;
uint32_t xcd_mapping(int kind, int64_t n, int64_t tpc, int64_t pool_blocks, int64_t chunk) {
  if (move_variant() & 0x2000000) return 0u;
  if (move_variant() & 0x4000000) return kXcdChunk;
  if (move_variant() & 0x8000000) return tpc % 2 == 0 ? kXcdPairs : 0u;
  if (n < 96 || tpc < 2 || kind == kMapDequant) return 0u;
  if (kind == kMapPoolToPool) return tpc >= 8 || tpc % 2 ? kXcdChunk : kXcdPairs;
  if (tpc % 2) return 0u;
  if (kind == kMapPack && (double)n * 2097152.0 > 1.25 * (double)pool_blocks * (double)chunk) return 0u;
  return kXcdPairs;
}

template <typename V, int U, int KIND, int ORDER, bool PAIRS, int POLICY>
void launch_move_full(const MoveArgs &a, uint32_t n, uint32_t order_arg, dim3 grid, bool full,
                      const PlaneTables<KIND == kPoolToPool ? 2 : 1> &t, hipStream_t s) {
  if (full)
    emm_block_move_kernel<V, U, KIND, ORDER, true, PAIRS, POLICY><<<grid, kThreads, 0, s>>>(
        a.idx_a, a.idx_b, a.lin, a.lin_plane_stride, a.chunk, a.src_nb, a.dst_nb, n, order_arg, t, NoIds{});
  else
    emm_block_move_kernel<V, U, KIND, ORDER, false, PAIRS, POLICY><<<grid, kThreads, 0, s>>>(
        a.idx_a, a.idx_b, a.lin, a.lin_plane_stride, a.chunk, a.src_nb, a.dst_nb, n, order_arg, t, NoIds{});
}

template <typename V, int U, int KIND, int POLICY>
void launch_move_inline(const MoveArgs &a, uint32_t n, uint32_t order_arg, dim3 grid, bool full,
                        const PlaneTables<1> &t, const InlineIds &ids, hipStream_t s) {
  if (full)
    emm_block_move_kernel<V, U, KIND, kOrderPlain, true, false, POLICY, true><<<grid, kThreads, 0, s>>>(
        nullptr, nullptr, a.lin, a.lin_plane_stride, a.chunk, a.src_nb, a.dst_nb, n, order_arg, t, ids);
  else
    emm_block_move_kernel<V, U, KIND, kOrderPlain, false, false, POLICY, true><<<grid, kThreads, 0, s>>>(
        nullptr, nullptr, a.lin, a.lin_plane_stride, a.chunk, a.src_nb, a.dst_nb, n, order_arg, t, ids);
}

template <int KIND, int ORDER, bool PAIRS>
void launch_move_vec(const MoveArgs &a, uint32_t n, uint32_t order_arg, dim3 grid, int vec, int policy, bool full,
                     const PlaneTables<KIND == kPoolToPool ? 2 : 1> &t, hipStream_t s) {
  // 16-byte lanes: one vector per lane, sc0 sc1 stores (nt stores in benchmark builds on request);
  // rare unaligned shapes: narrower lanes, four per lane, nt stores
  if (vec == 16 && policy == 1) launch_move_full<u32x4, 1, KIND, ORDER, PAIRS, 1>(a, n, order_arg, grid, full, t, s);
  else if (vec == 16) launch_move_full<u32x4, 1, KIND, ORDER, PAIRS, 0>(a, n, order_arg, grid, full, t, s);
  else if (vec == 4) launch_move_full<uint32_t, 4, KIND, ORDER, PAIRS, 0>(a, n, order_arg, grid, false, t, s);
  else if (vec == 2) launch_move_full<uint16_t, 4, KIND, ORDER, PAIRS, 0>(a, n, order_arg, grid, false, t, s);
  else launch_move_full<uint8_t, 4, KIND, ORDER, PAIRS, 0>(a, n, order_arg, grid, false, t, s);
}

int common_align(int a, const void *p) {
  int x = 16;
  while (x > 1 && !aligned(p, x)) x >>= 1;
  return a < x ? a : x;
}

int check_pool_args(const char *what, const void *const *layer_ptrs, int num_layers,
                    int num_kv, int64_t num_blocks, int64_t chunk_bytes, int64_t n) {
  if (num_layers < 0 || num_layers > EMM_MAX_LAYERS)
    return fail(EMM_EINVAL, "%s: num_layers=%d outside [0, %d]", what, num_layers, EMM_MAX_LAYERS);
  if (num_kv < 0 || num_blocks < 0 || chunk_bytes < 0 || n < 0)
    return fail(EMM_EINVAL, "%s: negative size (num_kv=%d num_blocks=%lld chunk_bytes=%lld n=%lld)",
                what, num_kv, (long long)num_blocks, (long long)chunk_bytes, (long long)n);
  if (num_blocks > 0x7fffffffLL)
    return fail(EMM_EINVAL, "%s: num_blocks=%lld exceeds 2^31-1", what, (long long)num_blocks);
  if (num_layers > 0 && !layer_ptrs) return fail(EMM_EINVAL, "%s: layer_ptrs is null", what);
  for (int l = 0; l < num_layers; ++l)
    if (!layer_ptrs[l] && n > 0 && num_blocks > 0)
      return fail(EMM_EINVAL, "%s: layer_ptrs[%d] is null", what, l);
  return EMM_OK;
}

// Build the plane tables for groups of at most kMaxPlanes (layer, kv) planes and launch, at most
// kMaxGridY blocks per launch. A null layer table means that side is the linear buffer
// [planes, n, chunk]. `pairs`: idx_a holds (src, dst) pairs (copy_blocks).
template <int KIND>
int move_planes(const void *const *src_layers, int64_t src_nb, void *const *dst_layers,
                int64_t dst_nb, int num_layers, int num_kv, int64_t chunk,
                const int64_t *idx_a, const int64_t *idx_b, bool pairs, int64_t n,
                const void *linear, hipStream_t s, const char *what, const int64_t *host_ids = nullptr) {
  constexpr bool SP = KIND != kUnpack, DP = KIND != kPack;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk == 0) return EMM_OK;
  InlineIds inline_ids;
  int al = 16;
  if (KIND != kPoolToPool) al = common_align(al, linear);
  for (int l = 0; l < num_layers; ++l) {
    if (SP) al = common_align(al, src_layers[l]);
    if (DP) al = common_align(al, dst_layers[l]);
  }
  // widest lane access that divides the chunk and every base address
  int vec = 16;
  while (vec > 1 && (chunk % vec != 0 || al % vec != 0)) vec >>= 1;
  if (vec == 8) vec = 4; // 8-byte lanes are not instantiated
  int policy = 1;
  if (vec == 16 && ((move_variant() >> 8) & 0xf) == 1) policy = 0;
  const int64_t tile_bytes = (int64_t)(vec == 16 ? 1 : 4) * kThreads * vec;
  const int64_t tpc = (chunk + tile_bytes - 1) / tile_bytes;
  if (tpc > 0x7fffffffLL)
    return fail(EMM_EINVAL, "%s: chunk of %lld bytes needs too many tiles", what, (long long)chunk);
  const bool full = chunk % tile_bytes == 0;

  const int64_t planes = (int64_t)num_layers * num_kv;
  for (int64_t pl0 = 0; pl0 < planes; pl0 += kMaxPlanes) {
    const int cnt = (int)((planes - pl0 < kMaxPlanes) ? (planes - pl0) : kMaxPlanes);
    PlaneTables<KIND == kPoolToPool ? 2 : 1> t;
    for (int i = 0; i < cnt; ++i) {
      const int64_t l = (pl0 + i) / num_kv, kv = (pl0 + i) % num_kv;
      if (SP) t.t[0].base[i] = (char *)src_layers[l] + kv * src_nb * chunk;
      if (DP) t.t[KIND == kPoolToPool ? 1 : 0].base[i] = (char *)dst_layers[l] + kv * dst_nb * chunk;
    }
    // blocks per launch: what the grid allows, or what the argument block holds (host tables)
    const int64_t step = host_ids ? EMM_MAX_INLINE_IDS : kMaxGridY;
    for (int64_t j0 = 0; j0 < n; j0 += step) {
      const int64_t ny = (n - j0 < step) ? (n - j0) : step;
      if (host_ids) { // ids travel in the argument block; what the device path would skip becomes the skip mark
        const int64_t nb = SP ? src_nb : dst_nb;
        for (int64_t j = 0; j < ny; ++j)
          inline_ids.id[j] = (host_ids[j0 + j] >= 0 && host_ids[j0 + j] < nb) ? (uint32_t)host_ids[j0 + j] : 0xffffffffu;
      }
      MoveArgs a;
      a.idx_a = idx_a ? idx_a + (pairs ? 2 * j0 : j0) : nullptr;
      a.idx_b = idx_b ? idx_b + j0 : nullptr;
      a.lin = linear ? (char *)linear + (pl0 * n + j0) * chunk : nullptr;
      a.lin_plane_stride = n * chunk;
      a.chunk = chunk;
      a.src_nb = (uint32_t)src_nb;
      a.dst_nb = (uint32_t)dst_nb;
      const uint32_t remap = xcd_mapping(KIND == kPoolToPool ? kMapPoolToPool : KIND == kPack ? kMapPack : kMapUnpack, ny, tpc,
                                          SP ? src_nb : dst_nb, chunk);
      if constexpr (KIND != kPoolToPool) {
        if (host_ids) { // at most EMM_MAX_INLINE_IDS blocks per launch, plain order
          const dim3 grid((uint32_t)tpc, (uint32_t)ny, (uint32_t)cnt);
          if (vec == 16) launch_move_inline<u32x4, 1, KIND, 1>(a, (uint32_t)ny, remap, grid, full, t, inline_ids, s);
          else if (vec == 4) launch_move_inline<uint32_t, 4, KIND, 0>(a, (uint32_t)ny, remap, grid, false, t, inline_ids, s);
          else if (vec == 2) launch_move_inline<uint16_t, 4, KIND, 0>(a, (uint32_t)ny, remap, grid, false, t, inline_ids, s);
          else launch_move_inline<uint8_t, 4, KIND, 0>(a, (uint32_t)ny, remap, grid, false, t, inline_ids, s);
          const int rc = check_launch(what);
          if (rc != EMM_OK) return rc;
          continue;
        }
      }
      if constexpr (KIND == kPoolToPool) {
        const uint32_t runs = (uint32_t)((ny + kRun - 1) / kRun);
        const dim3 grid((uint32_t)tpc, (uint32_t)(cnt * kRun), runs);
        if (pairs) launch_move_vec<KIND, kOrderRuns, true>(a, (uint32_t)ny, runs / cnt | remap, grid, vec, policy, full, t, s);
        else launch_move_vec<KIND, kOrderRuns, false>(a, (uint32_t)ny, runs / cnt | remap, grid, vec, policy, full, t, s);
      } else {
        // long scatters (unpack) are walked in groups of 256 blocks per plane visit (6712 blocks in one
        // launch: 6.41-6.50 TB/s; groups of 128: 6.16-6.29, of 512: 6.34, of 64: 5.73; plain order 6.40-6.46 on a
        // pool spread over the device but 5.65 on one that lies in one stretch of memory); short tables
        // already leave a plane after a few hundred blocks, and gathers (pack) measured faster in
        // the plain order
        int glog = (KIND == kUnpack && ny >= 1024) ? 8 : 0;
        const int forced = (move_variant() >> 16) & 0xf;
        if (forced) glog = forced == 0xf ? 0 : forced;
        if (glog > 0 && ((int64_t)cnt << glog) <= kMaxGridY) {
          const dim3 grid((uint32_t)tpc, (uint32_t)(cnt << glog), (uint32_t)((ny + (1 << glog) - 1) >> glog));
          launch_move_vec<KIND, kOrderGrouped, false>(a, (uint32_t)ny, (uint32_t)glog | (glog >= 3 ? remap : 0u), grid, vec, policy, full, t,
                                                          s);
        } else {
          const dim3 grid((uint32_t)tpc, (uint32_t)ny, (uint32_t)cnt);
          launch_move_vec<KIND, kOrderPlain, false>(a, (uint32_t)ny, remap, grid, vec, policy, full, t, s);
        }
      }
      const int rc = check_launch(what);
      if (rc != EMM_OK) return rc;
    }
  }
  return EMM_OK;
}

// ----------------------------------------------------------------------------
// fp8-e4m3fn <-> fp32 / 16-bit conversions (bit-exact integer formulations)
// ----------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) {
  return __uint_as_float(h << 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  _Float16 x;
  uint16_t b = (uint16_t)h;
  __builtin_memcpy(&x, &b, 2);
  return (float)x;
}

// fp32 -> e4m3fn with the rule of torch's cast: round to nearest even, no
// saturation; what rounds past 448 (464 is the tie that still gives 448), +-inf
// and NaN give sign|0x7F. gfx950's v_cvt_pk_fp8_f32 (OCP e4m3, overflow mode off)
// implements this for every non-NaN fp32 input and returns 0xFF for every NaN, so NaNs
// are first replaced by the infinity of their sign (the GPU tests compare the conversion
// with the oracle for every 16-bit input at many scales).
//
// Two overflow modes:
//   SAT = false  torch's x.to(float8_e4m3fn): overflow, +-inf and NaN -> sign|0x7F;
//   SAT = true   clamp(q, -448, 448) first (vLLM's fp8 KV-cache convention): overflow and
//                +-inf -> sign|0x7E (448), NaN stays NaN (sign|0x7F).
// finish_quotient prepares a quotient for the hardware conversion: |q| limited to inf
// (SAT: to 448) with one IEEE minimum — which also maps a NaN q to the limit, because the
// minimum returns its non-NaN operand —, `is_nan` (SAT only) puts the NaN back as an
// infinity, and the sign is taken from `sign_bits`.
template <bool SAT>
__device__ __forceinline__ float finish_quotient(float q, bool is_nan, uint32_t sign_bits) {
  float a = __builtin_fminf(__builtin_fabsf(q), SAT ? 448.0f : __builtin_inff());
  if constexpr (SAT) a = is_nan ? __builtin_inff() : a;
  return __uint_as_float(__float_as_uint(a) | (sign_bits & 0x80000000u));
}

__device__ __forceinline__ bool is_nan_bits(float f) { return (__float_as_uint(f) & 0x7fffffffu) > 0x7f800000u; }

// The rule in integer arithmetic, one value at a time (element-wise path); `f` has been
// through finish_quotient (no NaN).
__device__ __forceinline__ uint32_t f32_to_e4m3fn(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t sign = (u >> 24) & 0x80u;
  uint32_t a = u & 0x7fffffffu;
  uint32_t r;
  if (a >= 0x43f00000u) { // >= 480, inf
    r = 0x7fu;
  } else if (a < 0x3c800000u) { // below 2^-6: subnormal grid of 2^-9
    // |f| * 2^9 is exact; rintf rounds to nearest even; 8 encodes 2^-6
    r = (uint32_t)(int)__builtin_rintf(__uint_as_float(a) * 512.0f);
  } else {
    const uint32_t odd = (a >> 20) & 1u;
    a += 0x7ffffu + odd;    // RNE at bit 20
    a -= (120u << 23);      // rebias 127 -> 7
    r = a >> 20;            // may carry into 0x7f (NaN) for [464, 480)
  }
  return r | sign;
}

template <int SRC_DTYPE>
__device__ __forceinline__ float half_bits_to_f32(uint32_t h) {
  if constexpr (SRC_DTYPE == EMM_DTYPE_BF16)
    return bf16_bits_to_f32(h);
  else
    return f16_bits_to_f32(h);
}

// x / scale for a scale shared by a whole wave. The correctly rounded fp32 quotient is what
// torch's cast sees, so it must be reproduced bit for bit. For 2^-30 <= scale <= 2^30 it is
// obtained without the IEEE division sequence: with y = RN(1 / scale), q = RN(x * y),
// r = fma(-q, scale, x), the quotient is q' = fma(r, y, q). That q' equals RN(x / scale) for
// every input with at most 11 significant bits (all f16 and bf16 values) and every scale is
// established by exhaustion: the three operations commute with powers of two as long as nothing
// leaves the normal range, so the identity only depends on the two significands, and the GPU test
// suite checks all 2^10 x 2^23 significand pairs against the division (and, for what leaves the
// normal range, that the result still converts to the same byte). The correction step turns an
// infinite q (x infinite, or the product overflows) into a NaN and loses the sign of -0;
// finish_quotient repairs both, the sign of x being the sign of the quotient for a positive
// scale. Other scales (and negative ones) take the division.
struct Divisor {
  float scale;
  float recip;
  bool exact_fast;
};

__device__ __forceinline__ Divisor make_divisor(float scale, bool allow_fast) {
  Divisor d;
  d.scale = scale;
  d.recip = 1.0f / scale;
  d.exact_fast = allow_fast && scale >= 0x1p-30f && scale <= 0x1p30f;
  return d;
}

// the bare fast quotient (may be NaN where the division gives +-inf, see above)
__device__ __forceinline__ float divide_fast_raw(float x, const Divisor &d) {
  const float q = x * d.recip;
  const float r = __builtin_fmaf(-q, d.scale, x);
  return __builtin_fmaf(r, d.recip, q);
}

// x / scale, ready for the hardware conversion (no NaN, limited as the mode demands)
template <bool SAT>
__device__ __forceinline__ float divide_fast(float x, const Divisor &d) {
  return finish_quotient<SAT>(divide_fast_raw(x, d), is_nan_bits(x), __float_as_uint(x));
}

template <bool SAT>
__device__ __forceinline__ float divide_ieee(float x, float scale) {
  const float q = x / scale;
  return finish_quotient<SAT>(q, is_nan_bits(q), __float_as_uint(q));
}

// 8 sixteen-bit values (one u32x4) -> 8 e4m3fn bytes (one u32x2), q = rne(x / scale).
template <int SRC_DTYPE, bool SAT>
__device__ __forceinline__ u32x2 quant8(u32x4 in, const Divisor &d) {
  u32x2 out;
  if (d.exact_fast) {
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const uint32_t w0 = in[w * 2], w1 = in[w * 2 + 1];
      int r = 0;
      r = __builtin_amdgcn_cvt_pk_fp8_f32(divide_fast<SAT>(half_bits_to_f32<SRC_DTYPE>(w0 & 0xffffu), d),
                                          divide_fast<SAT>(half_bits_to_f32<SRC_DTYPE>(w0 >> 16), d), r, false);
      r = __builtin_amdgcn_cvt_pk_fp8_f32(divide_fast<SAT>(half_bits_to_f32<SRC_DTYPE>(w1 & 0xffffu), d),
                                          divide_fast<SAT>(half_bits_to_f32<SRC_DTYPE>(w1 >> 16), d), r, true);
      out[w] = (uint32_t)r;
    }
  } else {
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const uint32_t w0 = in[w * 2], w1 = in[w * 2 + 1];
      int r = 0;
      r = __builtin_amdgcn_cvt_pk_fp8_f32(divide_ieee<SAT>(half_bits_to_f32<SRC_DTYPE>(w0 & 0xffffu), d.scale),
                                          divide_ieee<SAT>(half_bits_to_f32<SRC_DTYPE>(w0 >> 16), d.scale), r, false);
      r = __builtin_amdgcn_cvt_pk_fp8_f32(divide_ieee<SAT>(half_bits_to_f32<SRC_DTYPE>(w1 & 0xffffu), d.scale),
                                          divide_ieee<SAT>(half_bits_to_f32<SRC_DTYPE>(w1 >> 16), d.scale), r, true);
      out[w] = (uint32_t)r;
    }
  }
  return out;
}

// one value, element-wise paths (always the division)
template <int SRC_DTYPE, bool SAT>
__device__ __forceinline__ uint8_t quant1(uint32_t h, float scale) {
  return (uint8_t)f32_to_e4m3fn(divide_ieee<SAT>(half_bits_to_f32<SRC_DTYPE>(h), scale));
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// two fp32 -> two 16-bit values in one dword, round to nearest even. The hardware
// conversions (v_cvt_pk_bf16_f32, v_cvt_f16_f32) equal the integer formulation for
// every non-NaN input (checked over all 2^32 bit patterns on the device); NaNs are
// replaced by the canonical quiet NaN by the caller.
template <int OUT_DTYPE>
__device__ __forceinline__ uint32_t pack16(float a, float b) {
  // The products must be rounded to fp32 before they are rounded to 16 bits: the
  // barrier stops the compiler from fusing multiply and convert into one
  // mixed-precision instruction with a single rounding.
  asm volatile("" : "+v"(a), "+v"(b));
  uint32_t r;
  if constexpr (OUT_DTYPE == EMM_DTYPE_BF16) {
    const bf16x2 h = __builtin_convertvector(f32x2{a, b}, bf16x2);
    __builtin_memcpy(&r, &h, 4);
  } else {
    const f16x2 h = __builtin_convertvector(f32x2{a, b}, f16x2);
    __builtin_memcpy(&r, &h, 4);
  }
  return r;
}

// 8 e4m3fn bytes (one u32x2) -> 8 sixteen-bit values (one u32x4):
// out = rne16(float(q) * scale); NaN bytes (0x7F / 0xFF) -> canonical quiet NaN.
// The byte -> fp32 step is v_cvt_pk_f32_fp8 (exact).
template <int OUT_DTYPE>
__device__ __forceinline__ u32x4 dequant8(u32x2 in, float scale) {
  constexpr uint32_t kNaN = OUT_DTYPE == EMM_DTYPE_BF16 ? 0x7fc0u : 0x7e00u;
  uint32_t o[4];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)in[w], false); // bytes 0, 1
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)in[w], true);  // bytes 2, 3
    o[w * 2] = pack16<OUT_DTYPE>(lo[0] * scale, lo[1] * scale);
    o[w * 2 + 1] = pack16<OUT_DTYPE>(hi[0] * scale, hi[1] * scale);
    // a byte is NaN iff its low 7 bits are all ones: rare, patched out of line
    const uint32_t nan = ((in[w] & 0x7f7f7f7fu) + 0x01010101u) & 0x80808080u;
    if (nan) {
      if (nan & 0x00000080u) o[w * 2] = (o[w * 2] & 0xffff0000u) | kNaN;
      if (nan & 0x00008000u) o[w * 2] = (o[w * 2] & 0x0000ffffu) | (kNaN << 16);
      if (nan & 0x00800000u) o[w * 2 + 1] = (o[w * 2 + 1] & 0xffff0000u) | kNaN;
      if (nan & 0x80000000u) o[w * 2 + 1] = (o[w * 2 + 1] & 0x0000ffffu) | (kNaN << 16);
    }
  }
  return u32x4{o[0], o[1], o[2], o[3]};
}

// ----------------------------------------------------------------------------
// dequant-unpack: fp8 transfer buffer -> 16-bit pool
// ----------------------------------------------------------------------------
struct LayerTable {
  char *base[EMM_MAX_LAYERS];
};

// One workgroup converts one tile of 4 KiB of fp8 bytes into 8 KiB. A wave owns 1 KiB of
// input: lane i loads bytes [8i, 8i+8) and [512+8i, 512+8i+8) and stores the two 16-byte
// results at twice those offsets, so that every load instruction covers 512 contiguous bytes
// and every store instruction 1 KiB of whole cache lines. Scalar arguments are explicit and
// ordered by first use (preloaded into scalar registers); the source does not depend on the
// block id, so it is loaded first and id, layer base and scale are waited for once.
// grid: x = tiles per chunk, y = blocks, z = 2 * layers (plain order), or the grouped order
// of the long unpack (GROUPED: y = plane * 2^g + position, z = group).
template <int OUT_DTYPE, bool GROUPED>
__global__ __launch_bounds__(kThreads) void emm_unpack_dequant_fp8_kernel(
    const char *__restrict__ packed, const int64_t *__restrict__ dst_idx, const float *__restrict__ k_scales,
    const float *__restrict__ v_scales, int64_t plane_stride /* n * chunk */, uint32_t chunk, uint32_t dst_nb,
    uint32_t n, uint32_t group_log2, const LayerTable layers) {
  constexpr uint32_t TILE = kThreads * 16;
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  xcd_map(group_log2, (chunk + TILE - 1) / TILE, GROUPED ? ~7u : (n & ~7u), bx, by); // as in emm_block_move_kernel
  group_log2 &= ~kXcdMask;
  uint32_t pl, j;
  if constexpr (GROUPED) {
    pl = by >> group_log2;
    j = (blockIdx.z << group_log2) + (by & ((1u << group_log2) - 1u));
    if (j >= n) return;
  } else {
    pl = blockIdx.z;
    j = by;
  }
  const uint32_t l = pl >> 1, kv = pl & 1;
  const uint32_t off0 = bx * TILE + wave * 1024 + lane * 8;
  const uint32_t off1 = off0 + 512;
  const bool live0 = off0 < chunk, live1 = off1 < chunk; // chunk is a multiple of 16
  const char *src = packed + (int64_t)pl * plane_stride + (uint64_t)j * chunk;
  const u32x2 a = ld<u32x2, true>(src + (live0 ? off0 : 0));
  const u32x2 c = ld<u32x2, true>(src + (live1 ? off1 : 0));
  int64_t b = dst_idx[j];
  char *dst_layer = layers.base[l];
  float scale = kv == 0 ? k_scales[l] : v_scales[l];
  asm volatile("" : "+s"(b), "+s"(dst_layer), "+s"(scale) : : "memory");
  if ((uint64_t)b >= (uint64_t)dst_nb) return;
  char *dst = dst_layer + ((uint64_t)kv * dst_nb + (uint64_t)b) * chunk * 2;
  if (live0) st_stream<u32x4, 1>(dst + (uint64_t)off0 * 2, dequant8<OUT_DTYPE>(a, scale));
  if (live1) st_stream<u32x4, 1>(dst + (uint64_t)off1 * 2, dequant8<OUT_DTYPE>(c, scale));
}

// ----------------------------------------------------------------------------
// reshape_and_cache: row scatter by slot_mapping
// ----------------------------------------------------------------------------
// Per-layer pointer tables of the whole-step launches (one launch for all layers).
struct AppendTables {
  const char *key[EMM_MAX_LAYERS];
  const char *value[EMM_MAX_LAYERS];
  char *key_cache[EMM_MAX_LAYERS];
  char *value_cache[EMM_MAX_LAYERS];
};
struct NoTables {};

constexpr int kWavesPerGroup = kThreads / 64;

// One wave moves R token rows, K and V both: the slot of a token is fetched once (a scalar load: the
// token index is wave-uniform) and 2 R sixteen-byte loads per lane are in flight before the first
// store. The source rows do not depend on the slots, so their loads are issued before the slots are
// waited for (rows of padded tokens are read and dropped). A model forward calls this once per layer
// with some tens of megabytes, where the time of a launch is its ramp: every scalar argument is an
// explicit kernel parameter, ordered by first use, so that the hardware has preloaded it into scalar
// registers when the wave starts (kernarg preload) and the first loads go out at once; small
// workgroups (one wave) start and drain fastest. TABLES: the four tensor pointers come from
// per-layer tables in the argument block instead (grid z = layer), one more scalar round trip.
// grid: x = groups of WAVES * R tokens, z = layers (TABLES) or 1.
template <typename V, int R, int WAVES, int POLICY, bool TABLES>
__global__ __launch_bounds__(WAVES * 64) void emm_append_kernel(
    const int64_t *__restrict__ slot_mapping, const char *key, const char *value, char *key_cache,
    char *value_cache, uint32_t num_tokens, uint32_t row_bytes, uint32_t key_stride, uint32_t value_stride,
    int64_t num_slots, const std::conditional_t<TABLES, AppendTables, NoTables> tables) {
  // (the 14 dwords up to value_stride are preloaded; num_slots is fetched while the loads are in flight)
  constexpr uint32_t VB = sizeof(V);
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = WAVES == 1 ? 0u : (uint32_t)__builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t t0 = (blockIdx.x * WAVES + wave) * R;
  if (t0 >= num_tokens) return;
  if constexpr (TABLES) {
    const uint32_t l = blockIdx.z;
    key = tables.key[l];
    value = tables.value[l];
    key_cache = tables.key_cache[l];
    value_cache = tables.value_cache[l];
  }
  int64_t slot[R];
#pragma unroll
  for (int r = 0; r < R; ++r) slot[r] = t0 + r < num_tokens ? slot_mapping[t0 + r] : -1;
  uint32_t off = lane * VB;
  const uint32_t o = off < row_bytes ? off : 0; // lanes past the row re-read its start; only stores are predicated
  V a[R], b[R];
  // Issue order (measured on a 28-layer chain of per-layer launches, 8448 tokens each; faster by 10 % than
  // issuing all loads first): rows of tokens 1.. go out at once and are in flight while the slots
  // arrive; token 0's rows are requested after the slot wait, and only if its slot is valid; then
  // stores in token order. The wave's reads and writes then overlap those of its neighbours instead
  // of the whole launch reading first and writing afterwards.
  // A whole-step launch (TABLES) is long enough to reach that overlap by itself and measured 3 %
  // faster with all rows requested before the slot wait; with one row per wave (launches of few
  // tokens) there is nothing to stagger and the row is requested at once.
  constexpr int kFirstEarly = (TABLES || R == 1) ? 0 : 1;
#pragma unroll
  for (int r = kFirstEarly; r < R; ++r) {
    const uint32_t t = t0 + r < num_tokens ? t0 + r : num_tokens - 1; // tail: re-read the last row, dropped below
    a[r] = ld_stream<V, POLICY>(key + (uint64_t)t * key_stride + o);
    b[r] = ld_stream<V, POLICY>(value + (uint64_t)t * value_stride + o);
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    asm volatile("" : "+s"(slot[r]) : : "memory");
    if ((uint64_t)slot[r] >= (uint64_t)num_slots) slot[r] = -1; // padding (< 0) and out-of-range slots: skipped
  }
  if constexpr (kFirstEarly == 1) {
    if (slot[0] >= 0) {
      a[0] = ld_stream<V, POLICY>(key + (uint64_t)t0 * key_stride + o);
      b[0] = ld_stream<V, POLICY>(value + (uint64_t)t0 * value_stride + o);
    }
  }
  if (off < row_bytes) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (slot[r] >= 0) {
        st_stream<V, POLICY>(key_cache + slot[r] * (int64_t)row_bytes + off, a[r]);
        st_stream<V, POLICY>(value_cache + slot[r] * (int64_t)row_bytes + off, b[r]);
      }
  }
  for (off += 64 * VB; off < row_bytes; off += 64 * VB) { // rows longer than 64 vectors
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (slot[r] >= 0) {
        a[r] = ld_stream<V, POLICY>(key + (uint64_t)(t0 + r) * key_stride + off);
        b[r] = ld_stream<V, POLICY>(value + (uint64_t)(t0 + r) * value_stride + off);
      }
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (slot[r] >= 0) {
        st_stream<V, POLICY>(key_cache + slot[r] * (int64_t)row_bytes + off, a[r]);
        st_stream<V, POLICY>(value_cache + slot[r] * (int64_t)row_bytes + off, b[r]);
      }
  }
}

// fp8 append: one wave quantises one token row of K or V (grid y = 2). VEC_ELEMS = 8: the row is
// converted in pieces of 1024 elements; lane i loads elements [8i, 8i+8) and [512+8i, 512+8i+8) of the
// piece (two 16-byte loads, each instruction 1 KiB contiguous) and stores the two 8-byte results at
// those element offsets (each instruction 512 contiguous bytes of whole cache lines). VEC_ELEMS = 1:
// element-wise path for rows that are not a multiple of 8 elements or misaligned bases. Scalar
// arguments are explicit and ordered by first use, as in emm_append_kernel. Strides and rows in
// elements. grid: x = groups of 4 tokens, y = 2 (K, V), z = layers (TABLES) or 1.
template <int SRC_DTYPE, int VEC_ELEMS, bool SAT, bool TABLES>
__global__ __launch_bounds__(kThreads) void emm_append_fp8_kernel(
    const int64_t *__restrict__ slot_mapping, const char *key, const char *value, uint32_t num_tokens,
    uint32_t row, uint32_t key_stride, uint32_t value_stride, const float *__restrict__ k_scales,
    const float *__restrict__ v_scales, char *key_cache, char *value_cache, int64_t num_slots, int32_t fast_div,
    const std::conditional_t<TABLES, AppendTables, NoTables> tables) {
  // (the 14 dwords up to v_scales are preloaded: everything the first loads need)
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t kv = blockIdx.y, l = TABLES ? blockIdx.z : 0;
  const uint32_t t = blockIdx.x * kWavesPerGroup + wave;
  if (t >= num_tokens) return;
  if constexpr (TABLES) {
    key = tables.key[l];
    value = tables.value[l];
    key_cache = tables.key_cache[l];
    value_cache = tables.value_cache[l];
  }
  const char *src = (kv == 0 ? key : value) + (uint64_t)t * (kv == 0 ? key_stride : value_stride) * 2;
  char *dst_base = kv == 0 ? key_cache : value_cache;
  int64_t slot = slot_mapping[t];
  const float scale = kv == 0 ? k_scales[l] : v_scales[l];

  if constexpr (VEC_ELEMS == 8) {
    uint32_t e0 = lane * 8, e1 = e0 + 512;
    // first piece: issued before slot and scale are waited for (rows of padded tokens are read and dropped)
    u32x4 a = ld<u32x4, true>(src + (e0 < row ? e0 : 0) * 2);
    u32x4 b = ld<u32x4, true>(src + (e1 < row ? e1 : 0) * 2);
    asm volatile("" : "+s"(slot) : : "memory");
    if ((uint64_t)slot >= (uint64_t)num_slots) return;
    const Divisor div = make_divisor(scale, fast_div != 0);
    char *dp = dst_base + slot * (int64_t)row;
    while (e0 < row) {
      const u32x2 qa = quant8<SRC_DTYPE, SAT>(a, div);
      const u32x2 qb = quant8<SRC_DTYPE, SAT>(b, div);
      st_stream<u32x2, 1>(dp + e0, qa);
      if (e1 < row) st_stream<u32x2, 1>(dp + e1, qb);
      e0 += 1024;
      e1 += 1024;
      if (e0 < row) {
        a = ld<u32x4, true>(src + e0 * 2);
        b = ld<u32x4, true>(src + (e1 < row ? e1 : e0) * 2);
      }
    }
  } else {
    if ((uint64_t)slot >= (uint64_t)num_slots) return;
    for (uint32_t e = lane; e < row; e += 64) {
      const uint16_t h = ld<uint16_t, false>(src + (int64_t)e * 2);
      st<uint8_t, false>(dst_base + slot * (int64_t)row + e, quant1<SRC_DTYPE, SAT>(h, scale));
    }
  }
}

int check_append_args(const char *what, const void *const *k, const void *const *v,
                      void *const *kc, void *const *vc, int num_layers,
                      const int64_t *slot_mapping, int64_t num_tokens, int64_t row,
                      int64_t ks, int64_t vs, int64_t num_slots) {
  if (num_layers < 0 || num_layers > EMM_MAX_LAYERS)
    return fail(EMM_EINVAL, "%s: num_layers=%d outside [0, %d]", what, num_layers, EMM_MAX_LAYERS);
  if (num_tokens < 0 || row < 0 || num_slots < 0 || ks < 0 || vs < 0)
    return fail(EMM_EINVAL, "%s: negative size", what);
  if (num_tokens == 0 || num_layers == 0 || row == 0) return EMM_OK;
  if (!slot_mapping) return fail(EMM_EINVAL, "%s: slot_mapping is null", what);
  if (!k || !v || !kc || !vc) return fail(EMM_EINVAL, "%s: pointer table is null", what);
  for (int l = 0; l < num_layers; ++l)
    if (!k[l] || !v[l] || !kc[l] || !vc[l])
      return fail(EMM_EINVAL, "%s: null tensor pointer at layer %d", what, l);
  if (ks < row || vs < row)
    return fail(EMM_EINVAL, "%s: token stride smaller than the row", what);
  if (num_tokens > 0x7fffffffLL) return fail(EMM_EINVAL, "%s: too many tokens", what);
  if (row > 0x7fffffffLL || ks > 0x7fffffffLL || vs > 0x7fffffffLL)
    return fail(EMM_EINVAL, "%s: row / token stride of 2 GiB or more", what);
  return EMM_OK;
}

void fill_tables(AppendTables &t, const void *const *k, const void *const *v, void *const *kc, void *const *vc,
                 int num_layers) {
  for (int l = 0; l < num_layers; ++l) {
    t.key[l] = (const char *)k[l];
    t.value[l] = (const char *)v[l];
    t.key_cache[l] = (char *)kc[l];
    t.value_cache[l] = (char *)vc[l];
  }
}

// launch shapes of the 16-byte copy append: (token rows per wave, waves per workgroup)
template <typename V, int R, int WAVES, int POLICY>
void launch_append(bool tables, const AppendTables &t, const int64_t *slot_mapping, int64_t num_tokens,
                   int64_t row_bytes, int64_t ks, int64_t vs, int64_t num_slots, int num_layers, hipStream_t s) {
  const int64_t per_group = (int64_t)R * WAVES;
  const uint32_t gx = (uint32_t)((num_tokens + per_group - 1) / per_group);
  if (tables)
    emm_append_kernel<V, R, WAVES, POLICY, true><<<dim3(gx, 1, (uint32_t)num_layers), WAVES * 64, 0, s>>>(
        slot_mapping, nullptr, nullptr, nullptr, nullptr, (uint32_t)num_tokens, (uint32_t)row_bytes, (uint32_t)ks,
        (uint32_t)vs, num_slots, t);
  else
    emm_append_kernel<V, R, WAVES, POLICY, false><<<dim3(gx), WAVES * 64, 0, s>>>(
        slot_mapping, t.key[0], t.value[0], t.key_cache[0], t.value_cache[0], (uint32_t)num_tokens,
        (uint32_t)row_bytes, (uint32_t)ks, (uint32_t)vs, num_slots, NoTables{});
}

int append_copy(const void *const *k, const void *const *v, void *const *kc, void *const *vc,
                int num_layers, const int64_t *slot_mapping, int64_t num_tokens,
                int64_t row_bytes, int64_t ks, int64_t vs, int64_t num_slots,
                bool tables, hipStream_t s, const char *what) {
  int rc = check_append_args(what, k, v, kc, vc, num_layers, slot_mapping, num_tokens,
                             row_bytes, ks, vs, num_slots);
  if (rc != EMM_OK) return rc;
  if (num_tokens == 0 || num_layers == 0 || row_bytes == 0) return EMM_OK;
  AppendTables t;
  fill_tables(t, k, v, kc, vc, num_layers);
  int al = 16;
  for (int l = 0; l < num_layers; ++l) {
    al = common_align(al, k[l]);
    al = common_align(al, v[l]);
    al = common_align(al, kc[l]);
    al = common_align(al, vc[l]);
  }
  int vec = al;
  while (vec > 1 && (row_bytes % vec || ks % vec || vs % vec)) vec >>= 1;
  if (vec == 16) {
    // workgroups of one wave start and drain fastest. A per-layer launch is best with four token rows
    // per wave (39.9 M tokens/s on the 28-layer chain of 8448-token launches; two rows 38.6, one 37.6),
    // a whole-step launch with one (6.23 TB/s; the others 6.11-6.14); the other shapes are selectable
    // in benchmark builds
    int shape = (move_variant() >> 12) & 0xf;
    // per-layer launches: as many waves as the tokens allow up to a few thousand (a decode step of 256 tokens:
    // 2.2 us per launch with one row per wave, 2.9 with four; the floor of an empty launch is 2.0)
    if (shape == 0) shape = tables ? 4 : num_tokens <= 1536 ? 4 : num_tokens <= 6144 ? 5 : 3;
    switch (shape) {
    case 1: launch_append<u32x4, 1, 4, 1>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    case 2: launch_append<u32x4, 2, 4, 1>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    case 4: launch_append<u32x4, 1, 1, 1>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    case 5: launch_append<u32x4, 2, 1, 1>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    default: launch_append<u32x4, 4, 1, 1>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    }
  } else {
    switch (vec) {
    case 8: launch_append<u32x2, 2, 4, 0>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    case 4: launch_append<uint32_t, 2, 4, 0>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    case 2: launch_append<uint16_t, 2, 4, 0>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    default: launch_append<uint8_t, 2, 4, 0>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, num_slots, num_layers, s); break;
    }
  }
  return check_launch(what);
}

template <int DT, int VEC, bool SAT>
void launch_append_fp8(bool tables, const AppendTables &t, const int64_t *slot_mapping, const float *k_scales,
                       const float *v_scales, int64_t num_tokens, int64_t row, int64_t ks, int64_t vs,
                       int64_t num_slots, int fast_div, int num_layers, hipStream_t s) {
  const uint32_t gx = (uint32_t)((num_tokens + kWavesPerGroup - 1) / kWavesPerGroup);
  if (tables)
    emm_append_fp8_kernel<DT, VEC, SAT, true><<<dim3(gx, 2, (uint32_t)num_layers), kThreads, 0, s>>>(
        slot_mapping, nullptr, nullptr, (uint32_t)num_tokens, (uint32_t)row, (uint32_t)ks, (uint32_t)vs, k_scales,
        v_scales, nullptr, nullptr, num_slots, fast_div, t);
  else
    emm_append_fp8_kernel<DT, VEC, SAT, false><<<dim3(gx, 2), kThreads, 0, s>>>(
        slot_mapping, t.key[0], t.value[0], (uint32_t)num_tokens, (uint32_t)row, (uint32_t)ks, (uint32_t)vs,
        k_scales, v_scales, t.key_cache[0], t.value_cache[0], num_slots, fast_div, NoTables{});
}

int append_fp8(const void *const *k, const void *const *v, void *const *kc, void *const *vc,
               int num_layers, const int64_t *slot_mapping, int64_t num_tokens,
               int64_t row_elems, int64_t ks, int64_t vs, int64_t num_slots,
               const float *k_scales, const float *v_scales, int src_dtype, bool tables,
               hipStream_t s, const char *what) {
  int rc = check_append_args(what, k, v, kc, vc, num_layers, slot_mapping, num_tokens,
                             row_elems, ks, vs, num_slots);
  if (rc != EMM_OK) return rc;
  const bool sat = (src_dtype & EMM_FP8_SATURATE) != 0;
  const int dt = src_dtype & ~EMM_FP8_SATURATE;
  if (dt != EMM_DTYPE_BF16 && dt != EMM_DTYPE_F16)
    return fail(EMM_EINVAL, "%s: unknown src_dtype %d", what, src_dtype);
  if (num_tokens == 0 || num_layers == 0 || row_elems == 0) return EMM_OK;
  if (!k_scales || !v_scales) return fail(EMM_EINVAL, "%s: scale pointer is null", what);
  AppendTables t;
  fill_tables(t, k, v, kc, vc, num_layers);
  int width = (row_elems % 8 || ks % 8 || vs % 8) ? 1 : 8;
  for (int l = 0; l < num_layers; ++l) {
    if (!aligned(k[l], 2) || !aligned(v[l], 2))
      return fail(EMM_EINVAL, "%s: 16-bit source not 2-byte aligned at layer %d", what, l);
    if (!aligned(k[l], 16) || !aligned(v[l], 16) || !aligned(kc[l], 8) || !aligned(vc[l], 8)) width = 1;
  }
  const int fast_div = (move_variant() & 0x1000000) ? 0 : 1;
#define EMM_FP8_LAUNCH(DT, VEC, SAT) \
  launch_append_fp8<DT, VEC, SAT>(tables, t, slot_mapping, k_scales, v_scales, num_tokens, row_elems, ks, vs, num_slots, fast_div, num_layers, s)
  if (dt == EMM_DTYPE_BF16) {
    if (width == 8) { if (sat) EMM_FP8_LAUNCH(EMM_DTYPE_BF16, 8, true); else EMM_FP8_LAUNCH(EMM_DTYPE_BF16, 8, false); }
    else { if (sat) EMM_FP8_LAUNCH(EMM_DTYPE_BF16, 1, true); else EMM_FP8_LAUNCH(EMM_DTYPE_BF16, 1, false); }
  } else {
    if (width == 8) { if (sat) EMM_FP8_LAUNCH(EMM_DTYPE_F16, 8, true); else EMM_FP8_LAUNCH(EMM_DTYPE_F16, 8, false); }
    else { if (sat) EMM_FP8_LAUNCH(EMM_DTYPE_F16, 1, true); else EMM_FP8_LAUNCH(EMM_DTYPE_F16, 1, false); }
  }
#undef EMM_FP8_LAUNCH
  return check_launch(what);
}

// ----------------------------------------------------------------------------
// reshape_and_cache, flash layout with free cache strides (e.g. the head-major
// pool [num_blocks, num_heads, block_size, head_size])
// ----------------------------------------------------------------------------
// One wave moves R token rows, K and V both, like emm_append_kernel (same leading arguments, preloaded; same
// issue order); each row is cut into heads, head h of slot (b, o) goes to
// cache + b * block_stride + o * page_stride + h * head_stride. No transpose happens below the
// size of a head row (256 bytes for head_size 128 in 16 bits), so no staging is needed: every
// store instruction still covers whole head rows. Block sizes and head rows that are powers of two
// (the usual case) are split with shifts; anything else with a division.
// A head-major pool takes 256-byte pieces 4 KiB apart and runs as fast as the contiguous layout
// (6.1 TB/s for 8448 tokens x 28 layers in one launch).
// grid: x = groups of R tokens, z = layers (TABLES) or 1.
template <typename V, int R, int POLICY, bool TABLES>
__global__ __launch_bounds__(64) void emm_append_strided_kernel(
    const int64_t *__restrict__ slot_mapping, const char *key, const char *value, char *key_cache,
    char *value_cache, uint32_t num_tokens, uint32_t row_bytes, uint32_t key_stride, uint32_t value_stride,
    uint32_t head_bytes, uint32_t block_size, int64_t num_slots, int64_t block_stride, int64_t page_stride,
    int64_t head_stride, const std::conditional_t<TABLES, AppendTables, NoTables> tables) {
  constexpr uint32_t VB = sizeof(V);
  const uint32_t lane = threadIdx.x;
  const uint32_t t0 = blockIdx.x * R;
  if (t0 >= num_tokens) return;
  if constexpr (TABLES) {
    const uint32_t l = blockIdx.z;
    key = tables.key[l];
    value = tables.value[l];
    key_cache = tables.key_cache[l];
    value_cache = tables.value_cache[l];
  }
  int64_t slot[R];
#pragma unroll
  for (int r = 0; r < R; ++r) slot[r] = t0 + r < num_tokens ? slot_mapping[t0 + r] : -1;
  uint32_t off = lane * VB;
  const uint32_t o = off < row_bytes ? off : 0; // lanes past the row re-read its start; only stores are predicated
  V a[R], b[R];
  constexpr int kFirstEarly = (TABLES || R == 1) ? 0 : 1; // as in emm_append_kernel
#pragma unroll
  for (int r = kFirstEarly; r < R; ++r) {
    const uint32_t t = t0 + r < num_tokens ? t0 + r : num_tokens - 1;
    a[r] = ld_stream<V, POLICY>(key + (uint64_t)t * key_stride + o);
    b[r] = ld_stream<V, POLICY>(value + (uint64_t)t * value_stride + o);
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    asm volatile("" : "+s"(slot[r]) : : "memory");
    if ((uint64_t)slot[r] >= (uint64_t)num_slots) slot[r] = -1; // padding (< 0) and out-of-range slots: skipped
  }
  if constexpr (kFirstEarly == 1) {
    if (slot[0] >= 0) {
      a[0] = ld_stream<V, POLICY>(key + (uint64_t)t0 * key_stride + o);
      b[0] = ld_stream<V, POLICY>(value + (uint64_t)t0 * value_stride + o);
    }
  }
  // where the rows start in the caches (wave-uniform), and the lane's place in the row's heads
  int64_t base[R];
  const bool bs_pow2 = (block_size & (block_size - 1)) == 0, head_pow2 = (head_bytes & (head_bytes - 1)) == 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t s = slot[r] < 0 ? 0 : slot[r];
    const int64_t blk = bs_pow2 ? s >> __builtin_ctz(block_size) : s / block_size;
    base[r] = blk * block_stride + (s - blk * block_size) * page_stride;
  }
  auto in_heads = [&](uint32_t byte) -> int64_t {
    const uint32_t h = head_pow2 ? byte >> __builtin_ctz(head_bytes) : byte / head_bytes;
    return (int64_t)h * head_stride + (byte - h * head_bytes);
  };
  if (off < row_bytes) {
    const int64_t w = in_heads(off);
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (slot[r] >= 0) {
        st_stream<V, POLICY>(key_cache + base[r] + w, a[r]);
        st_stream<V, POLICY>(value_cache + base[r] + w, b[r]);
      }
  }
  for (off += 64 * VB; off < row_bytes; off += 64 * VB) { // rows longer than 64 vectors
    const int64_t w = in_heads(off);
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (slot[r] >= 0) {
        a[r] = ld_stream<V, POLICY>(key + (uint64_t)(t0 + r) * key_stride + off);
        b[r] = ld_stream<V, POLICY>(value + (uint64_t)(t0 + r) * value_stride + off);
      }
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (slot[r] >= 0) {
        st_stream<V, POLICY>(key_cache + base[r] + w, a[r]);
        st_stream<V, POLICY>(value_cache + base[r] + w, b[r]);
      }
  }
}

template <typename V, int R, int POLICY>
void launch_append_strided(bool tables, const AppendTables &t, const int64_t *slot_mapping, int64_t num_tokens,
                           int64_t row_bytes, int64_t ks, int64_t vs, int64_t head_bytes, int block_size,
                           int64_t num_slots, int64_t block_stride, int64_t page_stride, int64_t head_stride,
                           int num_layers, hipStream_t s) {
  const uint32_t gx = (uint32_t)((num_tokens + R - 1) / R);
  if (tables)
    emm_append_strided_kernel<V, R, POLICY, true><<<dim3(gx, 1, (uint32_t)num_layers), 64, 0, s>>>(
        slot_mapping, nullptr, nullptr, nullptr, nullptr, (uint32_t)num_tokens, (uint32_t)row_bytes, (uint32_t)ks,
        (uint32_t)vs, (uint32_t)head_bytes, (uint32_t)block_size, num_slots, block_stride, page_stride, head_stride, t);
  else
    emm_append_strided_kernel<V, R, POLICY, false><<<dim3(gx), 64, 0, s>>>(
        slot_mapping, t.key[0], t.value[0], t.key_cache[0], t.value_cache[0], (uint32_t)num_tokens,
        (uint32_t)row_bytes, (uint32_t)ks, (uint32_t)vs, (uint32_t)head_bytes, (uint32_t)block_size, num_slots,
        block_stride, page_stride, head_stride, NoTables{});
}

int append_strided(const void *const *k, const void *const *v, void *const *kc, void *const *vc, int num_layers,
                   const int64_t *slot_mapping, int64_t num_tokens, int num_heads, int64_t head_bytes,
                   int block_size, int64_t num_blocks, int64_t ks, int64_t vs, int64_t block_stride,
                   int64_t page_stride, int64_t head_stride, hipStream_t s, const char *what) {
  if (num_layers < 0 || num_layers > EMM_MAX_LAYERS)
    return fail(EMM_EINVAL, "%s: num_layers=%d outside [0, %d]", what, num_layers, EMM_MAX_LAYERS);
  if (num_tokens < 0 || num_heads < 0 || head_bytes < 0 || block_size <= 0 || num_blocks < 0 || ks < 0 || vs < 0 ||
      block_stride < 0 || page_stride < 0 || head_stride < 0)
    return fail(EMM_EINVAL, "%s: negative size", what);
  const int64_t row_bytes = (int64_t)num_heads * head_bytes;
  if (num_tokens == 0 || row_bytes == 0 || num_layers == 0) return EMM_OK;
  if (head_bytes > 0x7fffffffLL || row_bytes > 0xffffffffLL) return fail(EMM_EINVAL, "%s: row too long", what);
  if (!k || !v || !kc || !vc || !slot_mapping) return fail(EMM_EINVAL, "%s: null pointer", what);
  if (ks < row_bytes || vs < row_bytes) return fail(EMM_EINVAL, "%s: token stride smaller than the row", what);
  if (head_stride < head_bytes || page_stride < head_bytes)
    return fail(EMM_EINVAL, "%s: head / page stride smaller than a head row", what);
  if (num_tokens > 0x7fffffffLL || ks > 0xffffffffLL || vs > 0xffffffffLL)
    return fail(EMM_EINVAL, "%s: too many tokens / token stride too large", what);
  AppendTables t;
  int al = 16;
  for (int l = 0; l < num_layers; ++l) {
    if (!k[l] || !v[l] || !kc[l] || !vc[l]) return fail(EMM_EINVAL, "%s: null tensor pointer at layer %d", what, l);
    al = common_align(al, k[l]);
    al = common_align(al, v[l]);
    al = common_align(al, kc[l]);
    al = common_align(al, vc[l]);
  }
  fill_tables(t, k, v, kc, vc, num_layers);
  int vec = al;
  while (vec > 1 && (head_bytes % vec || ks % vec || vs % vec || block_stride % vec || page_stride % vec ||
                     head_stride % vec))
    vec >>= 1;
  const bool tables = num_layers > 1;
  const int64_t num_slots = num_blocks * block_size;
#define EMM_STRIDED_LAUNCH(V_, R_, P_) \
  launch_append_strided<V_, R_, P_>(tables, t, slot_mapping, num_tokens, row_bytes, ks, vs, head_bytes, block_size, \
                                    num_slots, block_stride, page_stride, head_stride, num_layers, s)
  switch (vec) {
  case 16: // rows per wave as in the contiguous append
    if (tables || num_tokens <= 1536) EMM_STRIDED_LAUNCH(u32x4, 1, 1);
    else if (num_tokens <= 6144) EMM_STRIDED_LAUNCH(u32x4, 2, 1);
    else EMM_STRIDED_LAUNCH(u32x4, 4, 1);
    break;
  case 8: EMM_STRIDED_LAUNCH(u32x2, 1, 1); break;
  case 4: EMM_STRIDED_LAUNCH(uint32_t, 1, 0); break;
  case 2: EMM_STRIDED_LAUNCH(uint16_t, 1, 0); break;
  default: EMM_STRIDED_LAUNCH(uint8_t, 1, 0); break;
  }
#undef EMM_STRIDED_LAUNCH
  return check_launch(what);
}

// The quantising append for the same strided caches (an fp8 pool in the head-major layout): one wave quantises
// one token row of K or V (grid y = 2) exactly as emm_append_fp8_kernel does — 1024-element pieces, lane i converts
// elements [8 i, 8 i + 8) and [512 + 8 i, ...), the same quotient and conversion — and cuts the row into heads on
// the way out: element e of slot (b, o) goes to cache + b * block_stride + o * page_stride + (e / head_elems) *
// head_stride + e % head_elems (strides in bytes = elements). VEC_ELEMS = 8 needs head rows that are a multiple of
// 8 elements, so that an 8-byte store never crosses a head; VEC_ELEMS = 1 is the element-wise path for everything else.
template <int SRC_DTYPE, int VEC_ELEMS, bool SAT, bool TABLES>
__global__ __launch_bounds__(kThreads) void emm_append_strided_fp8_kernel(
    const int64_t *__restrict__ slot_mapping, const char *key, const char *value, uint32_t num_tokens,
    uint32_t row, uint32_t key_stride, uint32_t value_stride, const float *__restrict__ k_scales,
    const float *__restrict__ v_scales, char *key_cache, char *value_cache, uint32_t head_elems, uint32_t block_size,
    int64_t num_slots, int64_t block_stride, int64_t page_stride, int64_t head_stride, int32_t fast_div,
    const std::conditional_t<TABLES, AppendTables, NoTables> tables) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t kv = blockIdx.y, l = TABLES ? blockIdx.z : 0;
  const uint32_t t = blockIdx.x * kWavesPerGroup + wave;
  if (t >= num_tokens) return;
  if constexpr (TABLES) {
    key = tables.key[l];
    value = tables.value[l];
    key_cache = tables.key_cache[l];
    value_cache = tables.value_cache[l];
  }
  const char *src = (kv == 0 ? key : value) + (uint64_t)t * (kv == 0 ? key_stride : value_stride) * 2;
  char *dst_base = kv == 0 ? key_cache : value_cache;
  int64_t slot = slot_mapping[t];
  const float scale = kv == 0 ? k_scales[l] : v_scales[l];
  const bool head_pow2 = (head_elems & (head_elems - 1)) == 0;
  auto in_heads = [&](uint32_t e) -> int64_t {
    const uint32_t h = head_pow2 ? e >> __builtin_ctz(head_elems) : e / head_elems;
    return (int64_t)h * head_stride + (e - h * head_elems);
  };
  auto row_base = [&](int64_t s) -> char * {
    const int64_t blk = (block_size & (block_size - 1)) == 0 ? s >> __builtin_ctz(block_size) : s / block_size;
    return dst_base + blk * block_stride + (s - blk * block_size) * page_stride;
  };
  if constexpr (VEC_ELEMS == 8) {
    uint32_t e0 = lane * 8, e1 = e0 + 512;
    u32x4 a = ld<u32x4, true>(src + (e0 < row ? e0 : 0) * 2); // issued before slot and scale are waited for
    u32x4 b = ld<u32x4, true>(src + (e1 < row ? e1 : 0) * 2);
    asm volatile("" : "+s"(slot) : : "memory");
    if ((uint64_t)slot >= (uint64_t)num_slots) return;
    const Divisor div = make_divisor(scale, fast_div != 0);
    char *dp = row_base(slot);
    while (e0 < row) {
      const u32x2 qa = quant8<SRC_DTYPE, SAT>(a, div);
      const u32x2 qb = quant8<SRC_DTYPE, SAT>(b, div);
      st_stream<u32x2, 1>(dp + in_heads(e0), qa);
      if (e1 < row) st_stream<u32x2, 1>(dp + in_heads(e1), qb);
      e0 += 1024;
      e1 += 1024;
      if (e0 < row) {
        a = ld<u32x4, true>(src + e0 * 2);
        b = ld<u32x4, true>(src + (e1 < row ? e1 : e0) * 2);
      }
    }
  } else {
    if ((uint64_t)slot >= (uint64_t)num_slots) return;
    char *dp = row_base(slot);
    for (uint32_t e = lane; e < row; e += 64) {
      const uint16_t h = ld<uint16_t, false>(src + (int64_t)e * 2);
      st<uint8_t, false>(dp + in_heads(e), quant1<SRC_DTYPE, SAT>(h, scale));
    }
  }
}

template <int DT, int VEC, bool SAT>
void launch_append_strided_fp8(bool tables, const AppendTables &t, const int64_t *slot_mapping, const float *k_scales,
                               const float *v_scales, int64_t num_tokens, int64_t row, int64_t ks, int64_t vs,
                               int64_t head_elems, int block_size, int64_t num_slots, int64_t block_stride,
                               int64_t page_stride, int64_t head_stride, int fast_div, int num_layers, hipStream_t s) {
  const uint32_t gx = (uint32_t)((num_tokens + kWavesPerGroup - 1) / kWavesPerGroup);
  if (tables)
    emm_append_strided_fp8_kernel<DT, VEC, SAT, true><<<dim3(gx, 2, (uint32_t)num_layers), kThreads, 0, s>>>(
        slot_mapping, nullptr, nullptr, (uint32_t)num_tokens, (uint32_t)row, (uint32_t)ks, (uint32_t)vs, k_scales,
        v_scales, nullptr, nullptr, (uint32_t)head_elems, (uint32_t)block_size, num_slots, block_stride, page_stride,
        head_stride, fast_div, t);
  else
    emm_append_strided_fp8_kernel<DT, VEC, SAT, false><<<dim3(gx, 2), kThreads, 0, s>>>(
        slot_mapping, t.key[0], t.value[0], (uint32_t)num_tokens, (uint32_t)row, (uint32_t)ks, (uint32_t)vs, k_scales,
        v_scales, t.key_cache[0], t.value_cache[0], (uint32_t)head_elems, (uint32_t)block_size, num_slots,
        block_stride, page_stride, head_stride, fast_div, NoTables{});
}

int append_strided_fp8(const void *const *k, const void *const *v, void *const *kc, void *const *vc, int num_layers,
                       const int64_t *slot_mapping, int64_t num_tokens, int num_heads, int64_t head_elems,
                       int block_size, int64_t num_blocks, int64_t ks, int64_t vs, int64_t block_stride,
                       int64_t page_stride, int64_t head_stride, const float *k_scales, const float *v_scales,
                       int src_dtype, hipStream_t s, const char *what) {
  if (num_layers < 0 || num_layers > EMM_MAX_LAYERS)
    return fail(EMM_EINVAL, "%s: num_layers=%d outside [0, %d]", what, num_layers, EMM_MAX_LAYERS);
  if (num_tokens < 0 || num_heads < 0 || head_elems < 0 || block_size <= 0 || num_blocks < 0 || ks < 0 || vs < 0 ||
      block_stride < 0 || page_stride < 0 || head_stride < 0)
    return fail(EMM_EINVAL, "%s: negative size", what);
  const bool sat = (src_dtype & EMM_FP8_SATURATE) != 0;
  const int dt = src_dtype & ~EMM_FP8_SATURATE;
  if (dt != EMM_DTYPE_BF16 && dt != EMM_DTYPE_F16) return fail(EMM_EINVAL, "%s: unknown src_dtype %d", what, src_dtype);
  const int64_t row = (int64_t)num_heads * head_elems;
  if (num_tokens == 0 || row == 0 || num_layers == 0) return EMM_OK;
  if (head_elems > 0x7fffffffLL || row > 0x7fffffffLL) return fail(EMM_EINVAL, "%s: row too long", what);
  if (!k || !v || !kc || !vc || !slot_mapping) return fail(EMM_EINVAL, "%s: null pointer", what);
  if (!k_scales || !v_scales) return fail(EMM_EINVAL, "%s: scale pointer is null", what);
  if (ks < row || vs < row) return fail(EMM_EINVAL, "%s: token stride smaller than the row", what);
  if (head_stride < head_elems || page_stride < head_elems)
    return fail(EMM_EINVAL, "%s: head / page stride smaller than a head row", what);
  if (num_tokens > 0x7fffffffLL || ks > 0x7fffffffLL || vs > 0x7fffffffLL)
    return fail(EMM_EINVAL, "%s: too many tokens / token stride too large", what);
  AppendTables t;
  int width = (head_elems % 8 || ks % 8 || vs % 8 || block_stride % 8 || page_stride % 8 || head_stride % 8) ? 1 : 8;
  for (int l = 0; l < num_layers; ++l) {
    if (!k[l] || !v[l] || !kc[l] || !vc[l]) return fail(EMM_EINVAL, "%s: null tensor pointer at layer %d", what, l);
    if (!aligned(k[l], 2) || !aligned(v[l], 2))
      return fail(EMM_EINVAL, "%s: 16-bit source not 2-byte aligned at layer %d", what, l);
    if (!aligned(k[l], 16) || !aligned(v[l], 16) || !aligned(kc[l], 8) || !aligned(vc[l], 8)) width = 1;
  }
  fill_tables(t, k, v, kc, vc, num_layers);
  const bool tables = num_layers > 1;
  const int64_t num_slots = num_blocks * block_size;
  const int fast_div = (move_variant() & 0x1000000) ? 0 : 1;
#define EMM_SFP8_LAUNCH(DT, VEC, SAT) \
  launch_append_strided_fp8<DT, VEC, SAT>(tables, t, slot_mapping, k_scales, v_scales, num_tokens, row, ks, vs, head_elems, \
                                          block_size, num_slots, block_stride, page_stride, head_stride, fast_div, num_layers, s)
  if (dt == EMM_DTYPE_BF16) {
    if (width == 8) { if (sat) EMM_SFP8_LAUNCH(EMM_DTYPE_BF16, 8, true); else EMM_SFP8_LAUNCH(EMM_DTYPE_BF16, 8, false); }
    else { if (sat) EMM_SFP8_LAUNCH(EMM_DTYPE_BF16, 1, true); else EMM_SFP8_LAUNCH(EMM_DTYPE_BF16, 1, false); }
  } else {
    if (width == 8) { if (sat) EMM_SFP8_LAUNCH(EMM_DTYPE_F16, 8, true); else EMM_SFP8_LAUNCH(EMM_DTYPE_F16, 8, false); }
    else { if (sat) EMM_SFP8_LAUNCH(EMM_DTYPE_F16, 1, true); else EMM_SFP8_LAUNCH(EMM_DTYPE_F16, 1, false); }
  }
#undef EMM_SFP8_LAUNCH
  return check_launch(what);
}

// ----------------------------------------------------------------------------
// reshape_and_cache, paged-attention layout: the one place where source and
// destination layouts transpose, staged through LDS
// ----------------------------------------------------------------------------
// key_cache   [num_blocks, num_heads, head_size / x, block_size, x]   x = 16 / cache element bytes
// value_cache [num_blocks, num_heads, head_size, block_size]
// key / value [num_tokens, num_heads * head_size] (row stride given)
// For one block the K region is (row_elems / x) groups of [block_size][x] = block_size * 16 bytes,
// the V region is row_elems runs of block_size elements. A token contributes one 16-byte piece to
// every K group and one element to every V run, so tokens that fill a block in order produce
// contiguous output; a single token produces 16-byte (K) and element-sized (V) stores at a stride
// of block_size * 16 bytes resp. block_size elements.
constexpr int kPagedRun = 16;    // tokens of a whole run = rows staged through LDS = rows of a round of direct stores
constexpr int kPagedRows = 32;   // token positions a tile looks at: an owned run may reach 15 tokens past the tile
constexpr int kPagedSeg = 256;   // row elements per workgroup (template parameter SEG); 128 for short launches, see append_paged
constexpr int kPagedSegShort = 128;

// One workgroup handles the rows of up to 31 tokens x up to SEG (256 or 128) row elements of K or V.
//
// Runs. Consecutive tokens with consecutive slots inside one 16-slot-aligned window of a block
// form a run (at most 16 tokens). A run belongs to the tile its first token lies in, so a tile
// of TT tokens owns runs that may extend up to 15 tokens past its end, and leaves the
// head of a run that started in the previous tile to that tile: prompts written in order give
// whole 16-token runs no matter where they start in the token list. Wave 0 finds the runs in
// registers from the 32 slots after the tile start (lane = token position, three ballots) and
// leaves the result in LDS: where the whole run (16 tokens that fill a 16-slot window; at most
// one per tile) starts and lands, and a compact list of the other owned tokens. One wave only:
// the instructions of this step are a visible part of a launch that lasts a few microseconds.
//
// Rows. Item q of a round of 16 tokens is (row q / (SEG / 8), 16-byte source piece q % (SEG / 8)): two per thread
// for SEG = 256, one for SEG = 128.
//  * The whole run goes to LDS (quantised to e4m3fn on the way when the cache is fp8; rows padded
//    by 16 bytes so that a column walk touches every bank once), one row after the other, and,
//    after a barrier, to the cache. K: lane q moves (group q / 16, token q % 16), one 16-byte LDS
//    read and one 16-byte store; 16 neighbouring lanes cover one group, a wave instruction 1 KiB of
//    contiguous cache. V: lane q gathers one 16-byte piece of the run's [element][16 tokens] region
//    from a column of the tile (8 or 16 element-sized LDS reads).
//  * Every other owned token (decode tokens, heads and tails of prompts) skips the barrier: both rows
//    of a thread are requested together; K is stored straight from the registers as 16-byte (fp8
//    cache: 8-byte) pieces; V passes through rows of a second LDS tile that only the wave itself
//    reads back, so that a store instruction covers 64 consecutive elements of one token (64 sectors
//    in 16 consecutive lines). Each such store is a partial write of a 32-byte sector — what the
//    layout costs for tokens that do not fill a block.
// The scalar arguments are explicit and ordered by first use: the 14 dwords up to value_stride
// arrive preloaded in scalar registers.
// TT = tokens per tile (the runs that start in a tile are its own): 16, or 4 for launches of few tokens — a
// decode step's lone tokens then spread over four times as many compute units, whose rate of
// element-sized stores is what such a launch waits for; finding the runs four times as often costs
// long launches more than that gains.
// grid: x = token tiles, y = 2 * row segments (bit 0: K | V), z = layers.
template <int CE, int SRC_DTYPE, bool SAT, int TT, int SEG, bool TABLES>
__global__ __launch_bounds__(kThreads) void emm_append_paged_kernel(
    const int64_t *__restrict__ slot_mapping, const char *key, const char *value, char *key_cache,
    char *value_cache, uint32_t num_tokens, uint32_t row_elems, uint32_t key_stride, uint32_t value_stride,
    uint32_t block_size, uint32_t vec_src, int64_t num_blocks, const float *k_scales, const float *v_scales,
    const std::conditional_t<TABLES, AppendTables, NoTables> tables) {
  constexpr int X = 16 / CE;               // elements per 16-byte piece of the cache
  constexpr int ROW = SEG * CE + 16; // LDS row stride in bytes
  constexpr int kPieces = SEG / 8;   // 16-byte source pieces per full row
  constexpr int N = kPagedRun * kPieces / kThreads; // items per thread in a round of 16 tokens
  constexpr int kPass = kThreads / kPieces;         // rows the workgroup covers with one item per thread
  static_assert(SEG % 64 == 0 && N >= 1 && N * kPass == kPagedRun, "tile width");
  __shared__ __attribute__((aligned(16))) char tile[kPagedRun * ROW];  // the whole run
  __shared__ __attribute__((aligned(16))) char stage[kPagedRun * ROW]; // V rows of the other tokens, wave-private
  __shared__ int64_t s_blk[kPagedRows];                                  // the other owned tokens
  __shared__ int32_t s_off[kPagedRows];
  __shared__ int32_t s_pos[kPagedRows];
  __shared__ int64_t s_wblk; // block and first offset of the whole run
  __shared__ int32_t s_woff;
  __shared__ int32_t s_w0;    // token position of the whole run's first token, or -1
  __shared__ int32_t s_count; // other owned tokens
  const int tid = threadIdx.x;
  const uint32_t kv = blockIdx.y & 1u, seg = blockIdx.y >> 1;
  const uint32_t t0 = blockIdx.x * TT;
  const int bs = (int)block_size;

  // ---- wave 0: slots, runs, owned tokens ----
  if (tid < 64) {
    const int i = tid;
    int64_t s = -1, prev = -1;
    if (i < kPagedRows && t0 + i < num_tokens) {
      s = slot_mapping[t0 + i];
      if (t0 + i > 0) prev = slot_mapping[t0 + i - 1];
    }
    const bool valid = s >= 0 && s < num_blocks * bs;
    int64_t blk = 0;
    int32_t off = 0;
    if (valid) {
      if ((bs & (bs - 1)) == 0) { // wave-uniform
        blk = s >> __builtin_ctz(bs);
        off = (int32_t)s & (bs - 1);
      } else {
        blk = s / bs;
        off = (int32_t)(s - blk * bs);
      }
    }
    const bool cont = valid && s == prev + 1 && (off & 15) != 0; // continues the previous token's run
    const uint64_t starts = __ballot(!cont); // bit j: token j starts a run or is skipped (lanes >= 32: set)
    const uint64_t below = starts & ((2ull << i) - 1ull);
    const int head = below ? 63 - __builtin_clzll(below) : -1; // first token of this token's run
    const bool owned = valid && head >= 0 && head < TT;
    const uint64_t owned_mask = __ballot(owned);
    // a run of 16 tokens starts at a multiple of 16 slots; its V region is 16-byte aligned if the block's is
    const bool whole = owned && !cont && i < TT && ((bs * CE) & 15) == 0 &&
                       __builtin_ctzll(starts >> (i + 1)) + 1 == 16;
    const uint64_t whole_mask = __ballot(whole);
    const int w0 = whole_mask ? (int)__builtin_ctzll(whole_mask) : -1;
    const uint64_t other_mask = owned_mask & ~(w0 >= 0 ? 0xffffull << w0 : 0ull);
    if ((other_mask >> i) & 1ull) {
      const int r = __builtin_popcountll(other_mask & ((1ull << i) - 1ull));
      s_blk[r] = blk;
      s_off[r] = off;
      s_pos[r] = i;
    }
    if (i == (w0 >= 0 ? w0 : 0)) {
      s_wblk = blk;
      s_woff = off;
      s_w0 = w0;
      s_count = __builtin_popcountll(other_mask);
    }
  }
  if constexpr (TABLES) {
    const uint32_t l = blockIdx.z;
    key = tables.key[l];
    value = tables.value[l];
    key_cache = tables.key_cache[l];
    value_cache = tables.value_cache[l];
  }
  const uint32_t e0 = seg * SEG;
  const uint32_t left = row_elems - e0;
  const int seg_elems = left < SEG ? (int)left : SEG; // multiple of X
  const int pieces = seg_elems >> 3;
  const char *src = kv == 0 ? key : value;
  char *cache = kv == 0 ? key_cache : value_cache;
  const uint32_t stride = kv == 0 ? key_stride : value_stride;
  const int64_t groups_per_block = row_elems / X;
  float scale = 1.0f;
  if constexpr (CE == 1) scale = kv == 0 ? k_scales[blockIdx.z] : v_scales[blockIdx.z];
  const Divisor div = make_divisor(scale, true);
  __syncthreads();
  const int w0 = s_w0, count = s_count;
  if (w0 < 0 && count == 0) return;
  const int c = tid % kPieces < pieces ? tid % kPieces : 0; // lanes past the row re-read its start; nothing of theirs is stored
  const bool live = tid % kPieces < pieces;
  const int row0 = tid / kPieces; // rows of the thread's items in a round: row0 + kPass * it

  // One element of a source row that does not allow 16-byte loads, converted for the cache.
  auto slow_elem = [&](int pos, int e) -> uint32_t {
    const uint16_t h = ld<uint16_t, false>(src + ((uint64_t)(t0 + pos) * stride + e0 + e) * 2);
    if constexpr (CE == 1) return quant1<SRC_DTYPE, SAT>(h, scale);
    return h;
  };

  // ---- the whole run -> LDS ----
  if (w0 >= 0) {
    if (vec_src) {
      // one row after the other (the second request goes out when the first row has arrived): a launch for one
      // layer has every workgroup in the same phase, and spreading the requests measured faster than bunching them
#pragma unroll
      for (int it = 0; it < N; ++it) {
        u32x4 v = ld<u32x4, true>(src + ((uint64_t)(t0 + w0 + row0 + kPass * it) * stride + e0 + c * 8) * 2);
        asm volatile("" : "+v"(v));
        if (live) {
          char *dst = tile + (row0 + kPass * it) * ROW;
          if constexpr (CE == 2)
            *reinterpret_cast<u32x4 *>(dst + (tid % kPieces) * 16) = v;
          else
            *reinterpret_cast<u32x2 *>(dst + (tid % kPieces) * 8) = quant8<SRC_DTYPE, SAT>(v, div);
        }
      }
    } else {
      for (int r = 0; r < kPagedRun; ++r)
        for (int e = tid; e < seg_elems; e += kThreads) {
          const uint32_t a = slow_elem(w0 + r, e);
          if constexpr (CE == 2)
            *reinterpret_cast<uint16_t *>(tile + r * ROW + e * 2) = (uint16_t)a;
          else
            *reinterpret_cast<uint8_t *>(tile + r * ROW + e) = (uint8_t)a;
        }
    }
  }

  // ---- the other owned tokens: straight from the registers, 16 tokens per round ----
  for (int base = 0; base < count; base += kPagedRun) {
    if (vec_src) {
      u32x4 v[N];
      int64_t dblk[N];
      int doff[N];
#pragma unroll
      for (int it = 0; it < N; ++it) {
        const int r = base + row0 + kPass * it;
        const int rc = r < count ? r : count - 1; // rows past the list re-read its last row
        dblk[it] = s_blk[rc];
        doff[it] = s_off[rc];
        v[it] = ld<u32x4, true>(src + ((uint64_t)(t0 + s_pos[rc]) * stride + e0 + c * 8) * 2);
      }
      // Wait for all rows here: a wait placed after the first item's stores would also wait for those
      // stores (loads and stores share one in-order counter).
#pragma unroll
      for (int it = 0; it < N; ++it) asm volatile("" : "+v"(v[it]));
#pragma unroll
      for (int it = 0; it < N; ++it) {
        if (base + row0 + kPass * it >= count || !live) continue;
        const uint32_t e = e0 + (tid % kPieces) * 8; // first element of the piece
        u32x2 q8{0, 0};
        if constexpr (CE == 1) q8 = quant8<SRC_DTYPE, SAT>(v[it], div);
        if (kv == 0) {
          char *dst = cache + ((dblk[it] * groups_per_block + e / X) * bs + doff[it]) * 16;
          if constexpr (CE == 2)
            st_stream<u32x4, 1>(dst, v[it]);
          else
            st_stream<u32x2, 1>(dst + (e % X), q8);
        } else {
          // V: through the wave's own rows of the staging tile, so that a store instruction covers 64
          // consecutive elements of one token (64 sectors in 16 consecutive lines) instead of every eighth
          char *dst = stage + (row0 + kPass * it) * ROW;
          if constexpr (CE == 2)
            *reinterpret_cast<u32x4 *>(dst + (tid % kPieces) * 16) = v[it];
          else
            *reinterpret_cast<u32x2 *>(dst + (tid % kPieces) * 8) = q8;
        }
      }
      if (kv == 1) {
        // rows row0 + kPass * it of lanes 0-31 and 32-63: the wave wrote them itself and LDS keeps a wave's order;
        // the fence (wavefront scope: no cache action) keeps the compiler from moving the reads above the writes
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const int lane = tid & 63, first = (tid >> 6) * (64 / kPieces);
#pragma unroll
        for (int rr = 0; rr < N * (64 / kPieces); ++rr) {
          const int rl = first + (rr % (64 / kPieces)) + kPass * (rr / (64 / kPieces));
          if (base + rl >= count) continue;
          const int64_t rblk = s_blk[base + rl];
          const int roff = s_off[base + rl];
          char *dst = cache + ((rblk * row_elems + e0) * bs + roff) * CE;
#pragma unroll
          for (int m = 0; m < SEG / 64; ++m) {
            const int e = m * 64 + lane;
            if (e >= seg_elems) continue;
            // plain stores: the tokens of a partial run write neighbouring elements of the same sectors, which the
            // L2 merges before they go to memory (written through, a step with an 11-token tail wrote 1 % more)
            if constexpr (CE == 2)
              st<uint16_t, false>(dst + (int64_t)e * bs * 2, *reinterpret_cast<const uint16_t *>(stage + rl * ROW + e * 2));
            else
              st<uint8_t, false>(dst + (int64_t)e * bs, *reinterpret_cast<const uint8_t *>(stage + rl * ROW + e));
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront"); // the next round overwrites the rows
        __builtin_amdgcn_wave_barrier();
      }
    } else {
      const int end = base + kPagedRun < count ? base + kPagedRun : count;
      for (int r = base; r < end; ++r) {
        const int pos = s_pos[r];
        const int64_t dblk = s_blk[r];
        const int doff = s_off[r];
        for (int e = tid; e < seg_elems; e += kThreads) {
          const uint32_t a = slow_elem(pos, e);
          const uint32_t ee = e0 + e;
          char *dst = kv == 0 ? cache + ((dblk * groups_per_block + ee / X) * bs + doff) * 16 + (ee % X) * CE
                              : cache + ((dblk * row_elems + ee) * bs + doff) * CE;
          if constexpr (CE == 2)
            st<uint16_t, false>(dst, (uint16_t)a);
          else
            st<uint8_t, false>(dst, (uint8_t)a);
        }
      }
    }
  }
  if (w0 < 0) return; // no whole run in this tile (the same in every wave)

  __syncthreads();
  const int64_t wblk = s_wblk;
  const int woff = s_woff;
  if (kv == 0) {
    // ---- K, whole run: 16-byte pieces, token fastest ----
    const int groups = seg_elems / X;
    const int64_t g0 = e0 / X;
    for (int q = tid; q < groups * 16; q += kThreads) {
      const int g = q >> 4, r = q & 15;
      const u32x4 v = *reinterpret_cast<const u32x4 *>(tile + r * ROW + g * 16);
      st_stream<u32x4, 1>(cache + ((wblk * groups_per_block + g0 + g) * bs + woff + r) * 16, v);
    }
    return;
  }
  // ---- V, whole run: 16-byte pieces of the run's [element][16 tokens] region ----
  if constexpr (CE == 2) {
    // The transposing LDS read of gfx950 (ds_read_b64_tr_b16) does the [4 tokens][16 elements] ->
    // [16 elements][4 tokens] step by itself: in every group of 16 lanes, lane 4 j + q points at elements
    // c .. c + 3 of token j (c = first element of the group + 4 q), and lane l receives element
    // (first element + l) of tokens 0 .. 3. Two such reads give a lane 8 tokens of its element = 16 bytes.
    // Lanes 0-31 of a wave take tokens 0-7 of 32 consecutive elements, lanes 32-63 tokens 8-15 of the same
    // elements, so that one store instruction covers the 32 elements' 1 KiB of output completely (whole
    // sectors). Every lane stays active through the reads (its address serves other lanes).
    typedef short v4i16 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4i16 lds_v4i16;
    const int lane = tid & 63, half = lane >> 5, grp = (lane >> 4) & 1, sub = lane & 15;
    for (int q0 = (tid >> 6) * 32; q0 < seg_elems; q0 += (kThreads >> 6) * 32) {
      const char *from = tile + (8 * half + (sub >> 2)) * ROW + (q0 + 16 * grp + 4 * (sub & 3)) * 2;
      uint32_t w[4];
#pragma unroll
      for (int m = 0; m < 2; ++m) {
        const v4i16 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16 *)(from + 4 * m * ROW));
        w[2 * m] = (uint32_t)(uint16_t)r[0] | ((uint32_t)(uint16_t)r[1] << 16);
        w[2 * m + 1] = (uint32_t)(uint16_t)r[2] | ((uint32_t)(uint16_t)r[3] << 16);
      }
      const int e = q0 + 16 * grp + sub;
      if (e >= seg_elems) continue;
      char *dst = cache + ((wblk * row_elems + e0 + e) * bs + woff) * 2 + half * 16;
      st_stream<u32x4, 1>(dst, u32x4{w[0], w[1], w[2], w[3]});
    }
  } else {
    for (int e = tid; e < seg_elems; e += kThreads) {
      const char *col = tile + e;
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t x = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k)
          x |= (uint32_t) * reinterpret_cast<const uint8_t *>(col + (4 * j + k) * ROW) << (8 * k);
        w[j] = x;
      }
      char *dst = cache + ((wblk * row_elems + e0 + e) * bs + woff);
      st_stream<u32x4, 1>(dst, u32x4{w[0], w[1], w[2], w[3]});
    }
  }
}

// The paged-attention append for the usual shapes (16-bit cache, sources that allow 16-byte loads, block size a
// power of two >= 16): workgroups of ONE wave, no block barrier.
//
// A wave owns a tile of 16 token positions x COLS row elements of K and V (FUSED) or of one of them (grid: x = the
// waves of a tile, then the layers of a whole-step launch, tiles slowest; x runs fastest, so the waves of one tile
// are dispatched side by side).
//
// Who stores what. 16 consecutive tokens whose slots fill one 16-slot-aligned window of a block are a whole run;
// the run belongs to the tile its first token lies in (it may reach 15 tokens into the next tile). Every other
// valid token is stored by its own tile, one token at a time. Both decisions need nothing but the 48 slots
// around the tile: lane i (< 48) loads the slots of positions t0 - 16 + i and + 1, four lane compares become
// four 64-bit masks (valid, consecutive, aligned, not at a window start), and the rest is scalar bit arithmetic:
//   links   E = valid & valid >> 1 & consecutive & next-not-at-a-window-start        (bit p: p -> p + 1 is a link)
//   15 links in a row from p: four shift-and steps; W = those & valid & aligned      (bit p: a whole run starts)
//   bits 1..15 of W: a run of the previous tile covers this tile's tokens below that bit;
//   bits 16..31: this tile's own run (at most one: two starts are at least 16 apart).
// Every wave of a tile repeats this (a dozen vector and two dozen scalar instructions) instead of sharing it
// through LDS and a barrier.
//
// Whole run: the 16 rows x COLS elements go to a wave-private LDS tile (rows padded by 16 bytes) and come back
// transposed: K as 16-byte pieces, lane -> (group, token), every store instruction 1 KiB of contiguous cache;
// V through the transposing LDS read ds_read_b64_tr_b16, lanes 0-31 the tokens 0-7 and lanes 32-63 the tokens
// 8-15 of the same 32 elements, again 1 KiB of whole sectors per store instruction.
// Other tokens: lane -> (token, piece) loads the row piece; K is stored from the registers as 16-byte pieces (the
// token's slot comes from the lane that holds it, one ds_bpermute); V passes through the LDS tile so that a store
// instruction writes 64 (COLS = 32: 2 x 32) consecutive elements of a token — element-sized writes, each a write
// request of its own: what this layout costs for a token that does not fill a block.
//
// Measured on MI355X, Qwen2-7B rows, 28 layers (per-layer launches replayed from a HIP graph / one launch for all
// layers; the general kernel below and the flash-layout append on the same slots and memory beside it):
//   8192-token prompt of whole runs   8.4 us per launch, 149 us (6.3 TB/s)   general 8.0, 152   flash layout 7.0, 146
//   2048-token prompt of whole runs   3.7 us per launch                       general 4.1
//   256 single tokens                  4.7 us per launch, 35-39 us             general 4.6, 41     flash layout 2.2, 8
//   256 single tokens + the prompt    12.7-13.2 us per launch, 247-251 us     general 13.1-15.9, 246   flash 7.2, 151
// Whole runs move at the speed of the flash-layout append; what is left is the single tokens: each of a token's 512 V
// elements and 64 K pieces is a write request of its own, whatever kernel issues it (K alone: 2.2 us for the 256
// tokens, the launch floor; V alone: 4.6). Tried on the single tokens' V stores and not kept: reading the word first so
// that the line is valid in the L2 (256 tokens x 28 layers in one launch: 69 us against 43), merging with a pair of
// 32-bit atomics (151 us), write-through stores (45 us), and rewriting whole 32-byte sectors (read the element's 16
// tokens, replace one, write back, 16 loads in flight per lane; only safe where no other token of the call shares the
// 16-slot window): the mixed step in one launch 237 us against 251, but 31 us against 12.7 per layer and a decode step
// 10 us against 4.8 — the cost is not that the writes are partial. The tile order (tiles slowest, layers inside) is
// worth 4 % on the one-launch form. How many row elements a wave takes, and whether K and V share a wave, follows the
// launch size (append_paged below).
template <int COLS, bool FUSED, bool TABLES>
__global__ __launch_bounds__(64) void emm_append_paged_wave_kernel(
    const int64_t *__restrict__ slot_mapping, const char *key, const char *value, char *key_cache,
    char *value_cache, uint32_t num_tokens, uint32_t row_elems, uint32_t key_stride, uint32_t value_stride,
    uint32_t bs_log2, uint64_t num_slots, const std::conditional_t<TABLES, AppendTables, NoTables> tables) {
  constexpr int PC = COLS / 8;     // 16-byte source pieces per row segment
  constexpr int RPI = 64 / PC;     // token rows one load instruction covers
  constexpr int NL = 16 / RPI;     // load instructions for 16 rows
  constexpr int ROW = COLS * 2 + 16; // LDS row stride in bytes
  static_assert(COLS == 512 || COLS == 256 || COLS == 128 || COLS == 32, "column width");
  __shared__ __attribute__((aligned(16))) char tiles[FUSED ? 2 : 1][16 * ROW]; // FUSED: K, V
  char *const ktile = tiles[0];
  char *const vtile = tiles[FUSED ? 1 : 0];
  const uint32_t lane = threadIdx.x;
  // grid: x = the waves of a tile (FUSED: one per column, K and V both; else two per column, K | V in bit 0), then the
  // layers (TABLES), tiles slowest. Workgroups go to the 8 XCDs round-robin in dispatch order; rotating the assignment
  // by the tile index spreads the V waves of consecutive tiles over all XCDs (the single tokens of V are eight times
  // the write requests of K).
  const uint32_t tile_idx = TABLES ? blockIdx.z : blockIdx.y;
  const uint32_t rot_mask = bs_log2 >> 8;
  bs_log2 &= 0xffu;
  const uint32_t xi = rot_mask ? (blockIdx.x + tile_idx) & rot_mask : blockIdx.x;
  const uint32_t col = FUSED ? xi : xi >> 1;
  const bool do_k = FUSED || (xi & 1u) == 0, do_v = FUSED || (xi & 1u) != 0;
  const uint32_t t0 = tile_idx * 16u;

  // ---- the 48 slots around the tile -> whole runs and single tokens (wave-uniform) ----
  const int32_t pos = (int32_t)t0 - 16 + (int32_t)lane, last = (int32_t)num_tokens - 1;
  const int32_t p0 = pos < 0 ? 0 : pos > last ? last : pos;
  const int32_t p1 = pos + 1 < 0 ? 0 : pos + 1 > last ? last : pos + 1;
  const int64_t s = slot_mapping[p0];
  const int64_t sn = slot_mapping[p1];
  if constexpr (TABLES) {
    const uint32_t l = blockIdx.y;
    key = tables.key[l];
    value = tables.value[l];
    key_cache = tables.key_cache[l];
    value_cache = tables.value_cache[l];
  }
  const uint32_t e0 = col * COLS;
  const uint32_t col_elems = row_elems - e0 < (uint32_t)COLS ? row_elems - e0 : (uint32_t)COLS; // multiple of 8
  const uint32_t piece = lane % PC, rsub = lane / PC;
  const bool live = piece * 8 < col_elems;
  const uint32_t bs_mask = (1u << bs_log2) - 1u;
  const uint64_t groups_per_block = row_elems >> 3;
  const uint32_t col_off = (e0 + (live ? piece * 8 : 0)) * 2; // the lane's byte offset inside a source row
  // Short launches (COLS = 32: one load instruction covers the tile's 16 rows) request the tile's own rows before the
  // slots have arrived: they are what single tokens and a run that starts on the tile grid need, and a short launch
  // is one chain of memory round trips; a run that starts inside the tile loads its rows again.
  constexpr bool EARLY = NL == 1;
  u32x4 early_k{0, 0, 0, 0}, early_v{0, 0, 0, 0};
  if constexpr (EARLY) {
    const uint32_t tr = t0 + rsub <= (uint32_t)last ? t0 + rsub : (uint32_t)last;
    if (do_k) early_k = ld<u32x4, true>(key + (uint64_t)tr * key_stride * 2 + col_off);
    if (do_v) early_v = ld<u32x4, true>(value + (uint64_t)tr * value_stride * 2 + col_off);
  }
  const uint32_t slo = (uint32_t)s, snlo = (uint32_t)sn;
  const uint32_t lo = t0 == 0 ? 16u : 0u;                                    // positions below 0
  const uint32_t hi = num_tokens - t0 + 16u < 48u ? num_tokens - t0 + 16u : 48u; // positions past the last token
  const uint64_t in_range = ((1ull << hi) - 1ull) & ~((1ull << lo) - 1ull);
  const uint64_t valid = __ballot((uint64_t)s < num_slots) & in_range; // slots are below 2^32 (checked by the host)
  const uint64_t consecutive = __ballot(snlo == slo + 1u);
  const uint64_t next_inside = __ballot((snlo & 15u) != 0u);
  const uint64_t aligned16 = __ballot((slo & 15u) == 0u);
  uint64_t e = valid & (valid >> 1) & consecutive & next_inside;
  e &= e >> 1;
  e &= e >> 2;
  e &= e >> 4;
  e &= e >> 7; // bit p: the 15 links p .. p + 14 are all there
  const uint64_t starts = e & valid & aligned16;
  const uint32_t prev_run = (uint32_t)starts & 0xfffeu;
  const uint32_t own_run = (uint32_t)(starts >> 16) & 0xffffu;
  const int w0 = own_run ? __builtin_ctz(own_run) : -1;
  uint32_t lone = (uint32_t)(valid >> 16) & 0xffffu;
  if (prev_run) lone &= ~((1u << __builtin_ctz(prev_run)) - 1u);
  if (w0 >= 0) lone &= (1u << w0) - 1u;
  if (w0 < 0 && lone == 0) return;

  // ---- the whole run: K and V rows -> LDS -> caches ----
  if (w0 >= 0) {
    const uint32_t sw = (uint32_t)__builtin_amdgcn_readlane((int)slo, 16 + w0);
    const uint64_t wblk = sw >> bs_log2;
    const uint32_t woff = sw & bs_mask;
    u32x4 vk[NL], vv[NL];
    if (EARLY && w0 == 0) {
      vk[0] = early_k;
      vv[0] = early_v;
    } else {
      const char *krows = key + (uint64_t)(t0 + w0) * key_stride * 2 + col_off;
      const char *vrows = value + (uint64_t)(t0 + w0) * value_stride * 2 + col_off;
      if (do_k) {
#pragma unroll
        for (int k = 0; k < NL; ++k) vk[k] = ld<u32x4, true>(krows + (uint64_t)(k * RPI + rsub) * key_stride * 2);
      }
      if (do_v) {
#pragma unroll
        for (int k = 0; k < NL; ++k) vv[k] = ld<u32x4, true>(vrows + (uint64_t)(k * RPI + rsub) * value_stride * 2);
      }
    }
    if (live && do_k) {
#pragma unroll
      for (int k = 0; k < NL; ++k) *reinterpret_cast<u32x4 *>(ktile + (k * RPI + rsub) * ROW + piece * 16) = vk[k];
    }
    if (live && do_v) {
#pragma unroll
      for (int k = 0; k < NL; ++k) *reinterpret_cast<u32x4 *>(vtile + (k * RPI + rsub) * ROW + piece * 16) = vv[k];
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront"); // the wave reads what its other lanes wrote
    __builtin_amdgcn_wave_barrier();
    if (do_k) {
      // K: lane -> (group 4 j + lane / 16, token lane % 16): a store instruction covers 1 KiB of contiguous cache
      const uint32_t r = lane & 15;
      char *kdst = key_cache + (((wblk * groups_per_block + (e0 >> 3)) << bs_log2) + woff + r) * 16;
#pragma unroll
      for (int j = 0; j < PC / 4; ++j) {
        const uint32_t g = 4 * j + (lane >> 4);
        const u32x4 x = *reinterpret_cast<const u32x4 *>(ktile + r * ROW + g * 16);
        if (g * 8 < col_elems) st_stream<u32x4, 1>(kdst + ((uint64_t)g << bs_log2) * 16, x);
      }
    }
    if (do_v) {
      typedef short v4i16 __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) v4i16 lds_v4i16;
      const uint32_t half = lane >> 5, grp = (lane >> 4) & 1, sub = lane & 15;
      char *vdst = value_cache + (((wblk * row_elems + e0) << bs_log2) + woff) * 2 + half * 16;
#pragma unroll
      for (int q0 = 0; q0 < COLS; q0 += 32) {
        // in every group of 16 lanes, lane 4 j + q points at elements c .. c + 3 of token j and lane l receives
        // element l of tokens 0 .. 3: two reads give a lane 8 tokens of its element
        const char *from = vtile + (8 * half + (sub >> 2)) * ROW + (q0 + 16 * grp + 4 * (sub & 3)) * 2;
        uint32_t w[4];
#pragma unroll
        for (int m = 0; m < 2; ++m) {
          const v4i16 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16 *)(from + 4 * m * ROW));
          w[2 * m] = (uint32_t)(uint16_t)t[0] | ((uint32_t)(uint16_t)t[1] << 16);
          w[2 * m + 1] = (uint32_t)(uint16_t)t[2] | ((uint32_t)(uint16_t)t[3] << 16);
        }
        const uint32_t el = q0 + 16 * grp + sub;
        if (el < col_elems) st_stream<u32x4, 1>(vdst + ((uint64_t)el << bs_log2) * 2, u32x4{w[0], w[1], w[2], w[3]});
      }
    }
    if (lone == 0) return;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront"); // the V tile is reused below
    __builtin_amdgcn_wave_barrier();
  }

  // ---- the other tokens of the tile ----
  // lane -> (token k * RPI + rsub, piece); lanes whose token is not one of these re-read the first of them
  // (all loads are issued together and unconditionally; only what is kept is predicated)
  const uint32_t first_lone = (uint32_t)__builtin_ctz(lone);
  bool mine[NL];
  u32x4 xk[NL], xv[NL];
#pragma unroll
  for (int k = 0; k < NL; ++k) {
    const uint32_t row = k * RPI + rsub;
    mine[k] = ((lone >> row) & 1u) && live;
    if constexpr (EARLY) {
      xk[k] = early_k;
      xv[k] = early_v;
    } else {
      const uint64_t tr = t0 + (mine[k] ? row : first_lone);
      if (do_k) xk[k] = ld<u32x4, true>(key + tr * key_stride * 2 + col_off);
      if (do_v) xv[k] = ld<u32x4, true>(value + tr * value_stride * 2 + col_off);
    }
  }
  // K: 16-byte pieces straight from the registers; the slot of the lane's token is held by lane 16 + token
  if (do_k) {
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const uint32_t sl = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((16 + k * RPI + rsub) * 4), (int)slo);
      if (mine[k])
        st_stream<u32x4, 1>(key_cache + (((((uint64_t)(sl >> bs_log2)) * groups_per_block + (e0 >> 3) + piece) << bs_log2) +
                                         (sl & bs_mask)) * 16, xk[k]);
    }
  }
  if (!do_v) return;
  // V: through the LDS tile, one token at a time
#pragma unroll
  for (int k = 0; k < NL; ++k)
    if (mine[k]) *reinterpret_cast<u32x4 *>(vtile + (k * RPI + rsub) * ROW + piece * 16) = xv[k];
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
  for (uint32_t m = lone; m;) { // at most 16 rounds
    const int i0 = __builtin_ctz(m);
    m &= m - 1;
    if constexpr (COLS >= 64) {
      const uint64_t sl = (uint32_t)__builtin_amdgcn_readlane((int)slo, 16 + i0);
      char *dst = value_cache + ((((sl >> bs_log2) * row_elems + e0) << bs_log2) + (sl & bs_mask)) * 2;
      // plain stores: neighbouring tokens of a partial run write neighbouring elements of the same sectors, which
      // the L2 merges before they go to memory
      for (uint32_t el = lane; el < col_elems; el += 64)
        st<uint16_t, false>(dst + ((uint64_t)el << bs_log2) * 2, *reinterpret_cast<const uint16_t *>(vtile + i0 * ROW + el * 2));
    } else { // two tokens per store instruction
      int i1 = -1;
      if (m) {
        i1 = __builtin_ctz(m);
        m &= m - 1;
      }
      const uint32_t s0 = (uint32_t)__builtin_amdgcn_readlane((int)slo, 16 + i0);
      const uint32_t s1 = (uint32_t)__builtin_amdgcn_readlane((int)slo, 16 + (i1 < 0 ? i0 : i1));
      const bool upper = lane >= (uint32_t)COLS;
      const int i = upper ? i1 : i0;
      const uint64_t sl = upper ? s1 : s0;
      const uint32_t el = lane & (COLS - 1);
      if (i >= 0 && el < col_elems)
        st<uint16_t, false>(value_cache + ((((sl >> bs_log2) * row_elems + e0 + el) << bs_log2) + (sl & bs_mask)) * 2,
                            *reinterpret_cast<const uint16_t *>(vtile + i * ROW + el * 2));
    }
  }
}

int append_paged(const void *const *k, const void *const *v, void *const *kc, void *const *vc, int num_layers,
                 const int64_t *slot_mapping, int64_t num_tokens, int num_heads, int head_size,
                 int block_size, int64_t num_blocks, int64_t ks, int64_t vs, int src_dtype,
                 int cache_elem_bytes, const float *k_scales, const float *v_scales, hipStream_t s,
                 const char *what) {
  if (num_layers < 0 || num_layers > EMM_MAX_LAYERS)
    return fail(EMM_EINVAL, "%s: num_layers=%d outside [0, %d]", what, num_layers, EMM_MAX_LAYERS);
  if (num_tokens < 0 || num_heads < 0 || head_size < 0 || block_size <= 0 || num_blocks < 0 || ks < 0 || vs < 0)
    return fail(EMM_EINVAL, "%s: negative size", what);
  if (cache_elem_bytes != 1 && cache_elem_bytes != 2)
    return fail(EMM_EINVAL, "%s: cache_elem_bytes=%d, expected 2 (16-bit cache) or 1 (fp8 cache)", what,
                cache_elem_bytes);
  const bool sat = (src_dtype & EMM_FP8_SATURATE) != 0;
  src_dtype &= ~EMM_FP8_SATURATE;
  if (src_dtype != EMM_DTYPE_BF16 && src_dtype != EMM_DTYPE_F16)
    return fail(EMM_EINVAL, "%s: unknown src_dtype %d", what, src_dtype);
  const int x = 16 / cache_elem_bytes;
  if (head_size % x)
    return fail(EMM_EINVAL, "%s: head_size=%d is not a multiple of x=%d", what, head_size, x);
  const int64_t row_elems = (int64_t)num_heads * head_size;
  if (num_tokens == 0 || row_elems == 0 || num_layers == 0) return EMM_OK;
  if (!k || !v || !kc || !vc || !slot_mapping) return fail(EMM_EINVAL, "%s: null pointer", what);
  if (cache_elem_bytes == 1 && (!k_scales || !v_scales)) return fail(EMM_EINVAL, "%s: scale pointer is null", what);
  if (ks < row_elems || vs < row_elems) return fail(EMM_EINVAL, "%s: token stride smaller than the row", what);
  // tiles of 4 tokens for launches of at most 256 tokens (a decode step, 256 lone tokens: 4.6 us per launch against
  // 5.9 with tiles of 16; a 512-token prompt: 5.4 against 4.5 — three of four small tiles find nothing to do)
  int tile_tokens = num_tokens <= 256 ? 4 : 16;
  if (((move_variant() >> 20) & 3) == 1) tile_tokens = 16;
  if (((move_variant() >> 20) & 3) == 2) tile_tokens = 4;
  const int64_t tiles = (num_tokens + tile_tokens - 1) / tile_tokens;
  // Row elements per workgroup: 128 instead of 256 while the launch of one layer still fits the device at once
  // (2048 resident workgroups: 256 compute units x 8). Each thread then moves one 16-byte piece instead of two, one
  // memory round trip less per workgroup, and twice as many workgroups share the work: a 512 / 1000 / 2000 / 3000
  // token prompt of Qwen2-7B rows takes 2.97 / 3.47 / 4.04 / 5.03 us per layer against 3.28 / 3.96 / 4.61 / 5.24,
  // 64 lone tokens + a 1024-token prompt 4.40 against 5.30, 4096 tokens the same (5.62); beyond that the narrow tiles
  // need a second round of workgroups and lose (5000 tokens: 7.8 against 6.3 us). Launches for several layers keep 256.
  int seg_elems = kPagedSeg;
  if (!(num_layers > 1) && tiles * 2 * ((row_elems + kPagedSegShort - 1) / kPagedSegShort) <= 2048) seg_elems = kPagedSegShort;
  if (((move_variant() >> 22) & 3) == 1) seg_elems = kPagedSeg;
  if (((move_variant() >> 22) & 3) == 2 && num_layers == 1) seg_elems = kPagedSegShort;
  const int64_t segs = (row_elems + seg_elems - 1) / seg_elems;
  if (tiles > 0x7fffffffLL || segs * 2 > kMaxGridY) return fail(EMM_EINVAL, "%s: too many tokens / too long rows", what);
  if (num_tokens > 0x7fffffffLL || row_elems > 0x7fffffffLL || ks > 0xffffffffLL || vs > 0xffffffffLL)
    return fail(EMM_EINVAL, "%s: num_tokens / row / token stride too large", what);
  const bool tables = num_layers > 1;
  AppendTables t;
  uint32_t vec_src = ks % 8 == 0 && vs % 8 == 0;
  for (int l = 0; l < num_layers; ++l) {
    if (!k[l] || !v[l] || !kc[l] || !vc[l]) return fail(EMM_EINVAL, "%s: null tensor pointer at layer %d", what, l);
    if (!aligned(k[l], 2) || !aligned(v[l], 2))
      return fail(EMM_EINVAL, "%s: 16-bit source not 2-byte aligned at layer %d", what, l);
    if (!aligned(kc[l], 16) || !aligned(vc[l], 16))
      return fail(EMM_EINVAL, "%s: cache not 16-byte aligned at layer %d", what, l);
    if (!aligned(k[l], 16) || !aligned(v[l], 16)) vec_src = 0;
    if (tables) {
      t.key[l] = (const char *)k[l];
      t.value[l] = (const char *)v[l];
      t.key_cache[l] = (char *)kc[l];
      t.value_cache[l] = (char *)vc[l];
    }
  }
  // The usual shapes take the kernel of one-wave workgroups: 16-bit cache, 16-byte loads from the sources, block size
  // a power of two from 16 on, all slots below 2^32 (run finding compares the low words). Benchmark builds can force
  // the general kernel (bit 28), the column width (bits 29-30: 1 = 128, 2 = 32, 3 = 256) and K and V in one wave or
  // in two (bits 20-21: 1 / 2).
  const bool bs_pow2 = (block_size & (block_size - 1)) == 0;
  const int64_t wave_tiles = (num_tokens + 15) / 16;
  if (cache_elem_bytes == 2 && vec_src && bs_pow2 && block_size >= 16 && row_elems % 8 == 0 &&
      num_blocks * block_size <= 0xffffffffLL && wave_tiles <= kMaxGridY && !(move_variant() & 0x10000000)) {
    // How fat a wave is follows the launch: a wave moves 16 tokens x `cols` row elements of K, of V, or of both
    // (`fused`). Measured per layer on Qwen2-7B rows (512 elements), prompts of whole runs / off the tile grid / single
    // tokens only / 256 single tokens + a prompt, 256 .. 16384 tokens: up to about a thousand tokens the narrow
    // shape (32 elements, K and V in separate waves) wins wherever single tokens are involved (512 single tokens: 7.3 us
    // against 9.1; 256 + a prompt of 768: 6.4 against 7.1) and loses little on pure prompts (3.3 against 3.0); beyond,
    // 128 elements with K and V in one wave is the best or within 3 % of it everywhere (8192-token prompt 8.4 us,
    // 2048: 3.7 where the general kernel takes 4.1). 256-element waves bring a long prompt of whole runs to the
    // flash-layout append's 7.15 us but cost a step with single tokens 1.2 us; benchmark builds keep them.
    const int64_t per128 = (row_elems + 127) / 128;
    int cols = 128;
    bool fused = true;
    if (num_layers == 1 && wave_tiles * per128 < 256) {
      cols = 32;
      fused = false;
    }
    const int forced = (move_variant() >> 29) & 3; // benchmark builds: bits 29-30 the width, bits 20-21 K and V fused or not
    if (forced == 1) cols = 128;
    if (forced == 2) cols = 32;
    if (forced == 3) cols = 256;
    if (((move_variant() >> 20) & 3) == 1) fused = true;
    if (((move_variant() >> 20) & 3) == 2) fused = false;
    const int64_t ncols = (row_elems + cols - 1) / cols;
    const int64_t nxw = fused ? ncols : 2 * ncols;
    if (nxw <= 0x7fffffffLL) {
      const dim3 wgrid((uint32_t)nxw, tables ? (uint32_t)num_layers : (uint32_t)wave_tiles,
                       tables ? (uint32_t)wave_tiles : 1u);
      const uint32_t nx = (uint32_t)nxw;
      const uint32_t rot_mask = (nx & (nx - 1)) == 0 && nx <= 0x800000u ? nx - 1 : 0u;
      const uint32_t bs_log2 = (uint32_t)__builtin_ctz((unsigned)block_size) | (rot_mask << 8);
      const uint64_t num_slots = (uint64_t)num_blocks * (uint64_t)block_size;
#define EMM_PAGED_WAVE(COLS_, FUSED_) \
  do { \
    if (tables) \
      emm_append_paged_wave_kernel<COLS_, FUSED_, true><<<wgrid, 64, 0, s>>>( \
          slot_mapping, nullptr, nullptr, nullptr, nullptr, (uint32_t)num_tokens, (uint32_t)row_elems, (uint32_t)ks, \
          (uint32_t)vs, bs_log2, num_slots, t); \
    else \
      emm_append_paged_wave_kernel<COLS_, FUSED_, false><<<wgrid, 64, 0, s>>>( \
          slot_mapping, (const char *)k[0], (const char *)v[0], (char *)kc[0], (char *)vc[0], (uint32_t)num_tokens, \
          (uint32_t)row_elems, (uint32_t)ks, (uint32_t)vs, bs_log2, num_slots, NoTables{}); \
  } while (0)
#ifdef EMM_BENCH_HOOKS
      if (cols == 256) { if (fused) EMM_PAGED_WAVE(256, true); else EMM_PAGED_WAVE(256, false); }
      else if (cols == 128 && !fused) EMM_PAGED_WAVE(128, false);
      else if (cols == 32 && fused) EMM_PAGED_WAVE(32, true);
      else
#endif
      if (cols == 128) EMM_PAGED_WAVE(128, true);
      else EMM_PAGED_WAVE(32, false);
#undef EMM_PAGED_WAVE
      return check_launch(what);
    }
  }
  const dim3 grid((uint32_t)tiles, (uint32_t)(segs * 2), (uint32_t)num_layers);
#define EMM_PAGED_LAUNCH3(CE_, DT_, SAT_, TT_, SEG_) \
  emm_append_paged_kernel<CE_, DT_, SAT_, TT_, SEG_, false><<<grid, kThreads, 0, s>>>( \
      slot_mapping, (const char *)k[0], (const char *)v[0], (char *)kc[0], (char *)vc[0], (uint32_t)num_tokens, \
      (uint32_t)row_elems, (uint32_t)ks, (uint32_t)vs, (uint32_t)block_size, vec_src, num_blocks, k_scales, \
      v_scales, NoTables{})
#define EMM_PAGED_LAUNCH2(CE_, DT_, SAT_, TT_) \
  do { \
    if (tables) \
      emm_append_paged_kernel<CE_, DT_, SAT_, TT_, kPagedSeg, true><<<grid, kThreads, 0, s>>>( \
          slot_mapping, nullptr, nullptr, nullptr, nullptr, (uint32_t)num_tokens, (uint32_t)row_elems, (uint32_t)ks, \
          (uint32_t)vs, (uint32_t)block_size, vec_src, num_blocks, k_scales, v_scales, t); \
    else if (seg_elems == kPagedSegShort) \
      EMM_PAGED_LAUNCH3(CE_, DT_, SAT_, TT_, kPagedSegShort); \
    else \
      EMM_PAGED_LAUNCH3(CE_, DT_, SAT_, TT_, kPagedSeg); \
  } while (0)
#define EMM_PAGED_LAUNCH(CE_, DT_, SAT_) \
  do { \
    if (tile_tokens == 4) EMM_PAGED_LAUNCH2(CE_, DT_, SAT_, 4); \
    else EMM_PAGED_LAUNCH2(CE_, DT_, SAT_, 16); \
  } while (0)
  if (cache_elem_bytes == 2) EMM_PAGED_LAUNCH(2, EMM_DTYPE_BF16, false);
  else if (src_dtype == EMM_DTYPE_BF16 && !sat) EMM_PAGED_LAUNCH(1, EMM_DTYPE_BF16, false);
  else if (src_dtype == EMM_DTYPE_BF16) EMM_PAGED_LAUNCH(1, EMM_DTYPE_BF16, true);
  else if (!sat) EMM_PAGED_LAUNCH(1, EMM_DTYPE_F16, false);
  else EMM_PAGED_LAUNCH(1, EMM_DTYPE_F16, true);
#undef EMM_PAGED_LAUNCH
#undef EMM_PAGED_LAUNCH2
#undef EMM_PAGED_LAUNCH3
  return check_launch(what);
}

// ----------------------------------------------------------------------------
// concat_rows: ragged segments -> one contiguous buffer
// ----------------------------------------------------------------------------
constexpr int kSegGroup = 16; // segments per group of the two-level tile -> segment search
constexpr int kSegGroups = EMM_MAX_SEGMENTS / kSegGroup;
static_assert(kSegGroups * kSegGroup == EMM_MAX_SEGMENTS, "segment table must split into whole groups");

struct ConcatParams {
  const char *src[EMM_MAX_SEGMENTS];
  int64_t dst_off[EMM_MAX_SEGMENTS];
  int64_t nbytes[EMM_MAX_SEGMENTS];
  uint32_t tile_start[EMM_MAX_SEGMENTS]; // first tile of each segment; unused entries 0xFFFFFFFF
  uint32_t group_start[kSegGroups];      // tile_start[kSegGroup * g]
  char *dst;
};

template <typename V, int U>
__global__ __launch_bounds__(kThreads) void emm_concat_rows_kernel(const ConcatParams p) {
  constexpr int64_t TILE = (int64_t)U * kThreads * sizeof(V);
  const uint32_t w = blockIdx.x;
  // Wave-uniform search for the last segment whose first tile is <= w, as two rounds
  // of counting over small fixed tables (two dependent fetches of the argument block
  // instead of the seven of a binary search over 128 entries).
  int g = -1;
#pragma unroll
  for (int k = 0; k < kSegGroups; ++k) g += p.group_start[k] <= w ? 1 : 0;
  const uint32_t *ts = p.tile_start + g * kSegGroup;
  int i = -1;
#pragma unroll
  for (int k = 0; k < kSegGroup; ++k) i += ts[k] <= w ? 1 : 0;
  const int seg = g * kSegGroup + i;
  const int64_t off = (int64_t)(w - p.tile_start[seg]) * TILE;
  copy_tile<V, kThreads, U, sizeof(V) == 16 ? 1 : 0>(p.src[seg] + off, p.dst + p.dst_off[seg] + off,
                                                     p.nbytes[seg] - off);
}

hipStream_t as_stream(emm_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

} // namespace

// ============================================================================
// C ABI
// ============================================================================
extern "C" {

const char *emm_last_error(void) { return g_last_error; }
int emm_abi_version(void) { return EMM_KV_ABI_VERSION; }

int emm_kv_pack(const void *const *layer_ptrs, int num_layers, int num_kv,
                int64_t num_blocks, int64_t chunk_bytes, const int64_t *block_idx,
                int64_t n, void *packed, emm_stream_t stream) {
  int rc = check_pool_args("emm_kv_pack", layer_ptrs, num_layers, num_kv, num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!block_idx || !packed) return fail(EMM_EINVAL, "emm_kv_pack: null block_idx / packed");
  return move_planes<kPack>(layer_ptrs, num_blocks, nullptr, 0, num_layers, num_kv, chunk_bytes,
                            block_idx, nullptr, false, n, packed, as_stream(stream), "emm_kv_pack");
}

int emm_kv_unpack(void *const *layer_ptrs, int num_layers, int num_kv,
                  int64_t num_blocks, int64_t chunk_bytes, const int64_t *block_idx,
                  int64_t n, const void *packed, emm_stream_t stream) {
  int rc = check_pool_args("emm_kv_unpack", (const void *const *)layer_ptrs, num_layers, num_kv,
                           num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!block_idx || !packed) return fail(EMM_EINVAL, "emm_kv_unpack: null block_idx / packed");
  return move_planes<kUnpack>(nullptr, 0, layer_ptrs, num_blocks, num_layers, num_kv, chunk_bytes,
                              nullptr, block_idx, false, n, packed, as_stream(stream), "emm_kv_unpack");
}

int emm_kv_pack_host_ids(const void *const *layer_ptrs, int num_layers, int num_kv,
                         int64_t num_blocks, int64_t chunk_bytes, const int64_t *host_block_idx,
                         int64_t n, void *packed, emm_stream_t stream) {
  const char *what = "emm_kv_pack_host_ids";
  int rc = check_pool_args(what, layer_ptrs, num_layers, num_kv, num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!host_block_idx || !packed) return fail(EMM_EINVAL, "%s: null host_block_idx / packed", what);
  return move_planes<kPack>(layer_ptrs, num_blocks, nullptr, 0, num_layers, num_kv, chunk_bytes,
                            nullptr, nullptr, false, n, packed, as_stream(stream), what, host_block_idx);
}

int emm_kv_unpack_host_ids(void *const *layer_ptrs, int num_layers, int num_kv,
                           int64_t num_blocks, int64_t chunk_bytes, const int64_t *host_block_idx,
                           int64_t n, const void *packed, emm_stream_t stream) {
  const char *what = "emm_kv_unpack_host_ids";
  int rc = check_pool_args(what, (const void *const *)layer_ptrs, num_layers, num_kv, num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!host_block_idx || !packed) return fail(EMM_EINVAL, "%s: null host_block_idx / packed", what);
  return move_planes<kUnpack>(nullptr, 0, layer_ptrs, num_blocks, num_layers, num_kv, chunk_bytes,
                              nullptr, nullptr, false, n, packed, as_stream(stream), what, host_block_idx);
}

int emm_copy_blocks(void *const *layer_ptrs, int num_layers, int num_kv,
                    int64_t num_blocks, int64_t chunk_bytes,
                    const int64_t *block_mapping, int64_t num_pairs, emm_stream_t stream) {
  int rc = check_pool_args("emm_copy_blocks", (const void *const *)layer_ptrs, num_layers, num_kv,
                           num_blocks, chunk_bytes, num_pairs);
  if (rc != EMM_OK) return rc;
  if (num_pairs == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!block_mapping) return fail(EMM_EINVAL, "emm_copy_blocks: null block_mapping");
  return move_planes<kPoolToPool>((const void *const *)layer_ptrs, num_blocks, layer_ptrs, num_blocks,
                                  num_layers, num_kv, chunk_bytes, block_mapping, nullptr, true,
                                  num_pairs, nullptr, as_stream(stream), "emm_copy_blocks");
}

int emm_kv_migrate(const void *const *src_layer_ptrs, int64_t src_num_blocks,
                   void *const *dst_layer_ptrs, int64_t dst_num_blocks, int num_layers,
                   int num_kv, int64_t chunk_bytes, const int64_t *src_idx,
                   const int64_t *dst_idx, int64_t n, emm_stream_t stream) {
  int rc = check_pool_args("emm_kv_migrate", src_layer_ptrs, num_layers, num_kv, src_num_blocks,
                           chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  rc = check_pool_args("emm_kv_migrate", (const void *const *)dst_layer_ptrs, num_layers, num_kv,
                       dst_num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!src_idx || !dst_idx) return fail(EMM_EINVAL, "emm_kv_migrate: null index array");
  return move_planes<kPoolToPool>(src_layer_ptrs, src_num_blocks, dst_layer_ptrs, dst_num_blocks,
                                  num_layers, num_kv, chunk_bytes, src_idx, dst_idx, false, n, nullptr,
                                  as_stream(stream), "emm_kv_migrate");
}

int emm_stream_copy(const void *src, void *dst, int64_t nbytes, emm_stream_t stream) {
  if (nbytes < 0) return fail(EMM_EINVAL, "emm_stream_copy: negative size");
  if (nbytes == 0) return EMM_OK;
  if (!src || !dst) return fail(EMM_EINVAL, "emm_stream_copy: null pointer");
  int vec = common_align(common_align(16, src), dst);
  while (vec > 1 && nbytes % vec) vec >>= 1;
  if (vec == 8) vec = 4;
  const int64_t tile = (int64_t)(vec == 16 ? 1 : 4) * kThreads * vec;
  const int64_t tiles = (nbytes + tile - 1) / tile;
  if (tiles > 0x7fffffffLL) return fail(EMM_EINVAL, "emm_stream_copy: %lld bytes need too many tiles", (long long)nbytes);
  const dim3 grid((uint32_t)tiles);
  hipStream_t s = as_stream(stream);
  const char *a = (const char *)src;
  char *b = (char *)dst;
  switch (vec) {
  case 16: emm_stream_copy_kernel<u32x4, 1, 1><<<grid, kThreads, 0, s>>>(a, b, nbytes); break;
  case 4: emm_stream_copy_kernel<uint32_t, 4, 0><<<grid, kThreads, 0, s>>>(a, b, nbytes); break;
  case 2: emm_stream_copy_kernel<uint16_t, 4, 0><<<grid, kThreads, 0, s>>>(a, b, nbytes); break;
  default: emm_stream_copy_kernel<uint8_t, 4, 0><<<grid, kThreads, 0, s>>>(a, b, nbytes); break;
  }
  return check_launch("emm_stream_copy");
}

int emm_kv_unpack_dequant_fp8(void *const *layer_ptrs, int num_layers, int64_t num_blocks,
                              int64_t chunk_elems, const int64_t *block_idx, int64_t n,
                              const void *packed_fp8, const float *k_scales,
                              const float *v_scales, int out_dtype, emm_stream_t stream) {
  const char *what = "emm_kv_unpack_dequant_fp8";
  int rc = check_pool_args(what, (const void *const *)layer_ptrs, num_layers, 2, num_blocks,
                           chunk_elems, n);
  if (rc != EMM_OK) return rc;
  if (out_dtype != EMM_DTYPE_BF16 && out_dtype != EMM_DTYPE_F16)
    return fail(EMM_EINVAL, "%s: unknown out_dtype %d", what, out_dtype);
  if (n == 0 || num_layers == 0 || chunk_elems == 0) return EMM_OK;
  if (!block_idx || !packed_fp8 || !k_scales || !v_scales)
    return fail(EMM_EINVAL, "%s: null pointer argument", what);
  if (chunk_elems % 16 != 0 || !aligned(packed_fp8, 16))
    return fail(EMM_EINVAL, "%s: chunk_elems (%lld) and packed_fp8 must be multiples of 16",
                what, (long long)chunk_elems);
  if (chunk_elems > 0x3fffffffLL || num_blocks > 0x7fffffffLL)
    return fail(EMM_EINVAL, "%s: chunk_elems / num_blocks too large", what);
  LayerTable t;
  for (int l = 0; l < num_layers; ++l) {
    if (!aligned(layer_ptrs[l], 16))
      return fail(EMM_EINVAL, "%s: layer_ptrs[%d] not 16-byte aligned", what, l);
    t.base[l] = (char *)layer_ptrs[l];
  }
  const int64_t tile = (int64_t)kThreads * 16;
  const int64_t tpc = (chunk_elems + tile - 1) / tile;
  hipStream_t s = as_stream(stream);
  for (int64_t j0 = 0; j0 < n; j0 += kMaxGridY) {
    const int64_t ny = (n - j0 < kMaxGridY) ? (n - j0) : kMaxGridY;
    const char *packed = (const char *)packed_fp8 + j0 * chunk_elems;
    const int64_t *idx = block_idx + j0;
    const int64_t stride = n * chunk_elems;
    const bool grouped = ny >= 1024 && ((2 * num_layers) << 8) <= kMaxGridY; // groups of 256 blocks, as in unpack
    const uint32_t remap = xcd_mapping(kMapDequant, ny, tpc, num_blocks, 2 * chunk_elems);
    const dim3 grid = grouped ? dim3((uint32_t)tpc, (uint32_t)((2 * num_layers) << 8), (uint32_t)((ny + 255) >> 8))
                              : dim3((uint32_t)tpc, (uint32_t)ny, (uint32_t)(2 * num_layers));
#define EMM_DQ_LAUNCH(DT, G) \
  emm_unpack_dequant_fp8_kernel<DT, G><<<grid, kThreads, 0, s>>>(packed, idx, k_scales, v_scales, stride, \
      (uint32_t)chunk_elems, (uint32_t)num_blocks, (uint32_t)ny, 8u | remap, t)
    if (out_dtype == EMM_DTYPE_BF16) { if (grouped) EMM_DQ_LAUNCH(EMM_DTYPE_BF16, true); else EMM_DQ_LAUNCH(EMM_DTYPE_BF16, false); }
    else { if (grouped) EMM_DQ_LAUNCH(EMM_DTYPE_F16, true); else EMM_DQ_LAUNCH(EMM_DTYPE_F16, false); }
#undef EMM_DQ_LAUNCH
    const int rc2 = check_launch(what);
    if (rc2 != EMM_OK) return rc2;
  }
  return EMM_OK;
}

int emm_reshape_and_cache(const void *key, const void *value, void *key_cache,
                          void *value_cache, const int64_t *slot_mapping,
                          int64_t num_tokens, int64_t row_bytes, int64_t key_stride_bytes,
                          int64_t value_stride_bytes, int64_t num_slots, emm_stream_t stream) {
  return append_copy(&key, &value, &key_cache, &value_cache, 1, slot_mapping, num_tokens,
                     row_bytes, key_stride_bytes, value_stride_bytes, num_slots, false,
                     as_stream(stream), "emm_reshape_and_cache");
}

int emm_reshape_and_cache_layers(const void *const *key_ptrs, const void *const *value_ptrs,
                                 void *const *key_cache_ptrs, void *const *value_cache_ptrs,
                                 int num_layers, const int64_t *slot_mapping,
                                 int64_t num_tokens, int64_t row_bytes,
                                 int64_t key_stride_bytes, int64_t value_stride_bytes,
                                 int64_t num_slots, emm_stream_t stream) {
  return append_copy(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers,
                     slot_mapping, num_tokens, row_bytes, key_stride_bytes, value_stride_bytes,
                     num_slots, true, as_stream(stream), "emm_reshape_and_cache_layers");
}

int emm_reshape_and_cache_fp8(const void *key, const void *value, void *key_cache,
                              void *value_cache, const int64_t *slot_mapping,
                              int64_t num_tokens, int64_t row_elems, int64_t key_stride_elems,
                              int64_t value_stride_elems, int64_t num_slots,
                              const float *k_scale, const float *v_scale, int src_dtype,
                              emm_stream_t stream) {
  return append_fp8(&key, &value, &key_cache, &value_cache, 1, slot_mapping, num_tokens,
                    row_elems, key_stride_elems, value_stride_elems, num_slots, k_scale, v_scale,
                    src_dtype, false, as_stream(stream), "emm_reshape_and_cache_fp8");
}

int emm_reshape_and_cache_fp8_layers(const void *const *key_ptrs, const void *const *value_ptrs,
                                     void *const *key_cache_ptrs, void *const *value_cache_ptrs,
                                     int num_layers, const int64_t *slot_mapping,
                                     int64_t num_tokens, int64_t row_elems,
                                     int64_t key_stride_elems, int64_t value_stride_elems,
                                     int64_t num_slots, const float *k_scales,
                                     const float *v_scales, int src_dtype, emm_stream_t stream) {
  return append_fp8(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers,
                    slot_mapping, num_tokens, row_elems, key_stride_elems, value_stride_elems,
                    num_slots, k_scales, v_scales, src_dtype, true, as_stream(stream),
                    "emm_reshape_and_cache_fp8_layers");
}

int emm_reshape_and_cache_strided(const void *const *key_ptrs, const void *const *value_ptrs,
                                  void *const *key_cache_ptrs, void *const *value_cache_ptrs,
                                  int num_layers, const int64_t *slot_mapping, int64_t num_tokens,
                                  int num_heads, int64_t head_bytes, int block_size, int64_t num_blocks,
                                  int64_t key_stride_bytes, int64_t value_stride_bytes,
                                  int64_t block_stride_bytes, int64_t page_stride_bytes,
                                  int64_t head_stride_bytes, emm_stream_t stream) {
  return append_strided(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers, slot_mapping,
                        num_tokens, num_heads, head_bytes, block_size, num_blocks, key_stride_bytes,
                        value_stride_bytes, block_stride_bytes, page_stride_bytes, head_stride_bytes,
                        as_stream(stream), "emm_reshape_and_cache_strided");
}

int emm_reshape_and_cache_strided_fp8(const void *const *key_ptrs, const void *const *value_ptrs,
                                      void *const *key_cache_ptrs, void *const *value_cache_ptrs, int num_layers,
                                      const int64_t *slot_mapping, int64_t num_tokens, int num_heads,
                                      int64_t head_elems, int block_size, int64_t num_blocks,
                                      int64_t key_stride_elems, int64_t value_stride_elems,
                                      int64_t block_stride_bytes, int64_t page_stride_bytes,
                                      int64_t head_stride_bytes, const float *k_scales, const float *v_scales,
                                      int src_dtype, emm_stream_t stream) {
  return append_strided_fp8(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers, slot_mapping,
                            num_tokens, num_heads, head_elems, block_size, num_blocks, key_stride_elems,
                            value_stride_elems, block_stride_bytes, page_stride_bytes, head_stride_bytes, k_scales,
                            v_scales, src_dtype, as_stream(stream), "emm_reshape_and_cache_strided_fp8");
}

int emm_reshape_and_cache_paged(const void *key, const void *value, void *key_cache, void *value_cache,
                                const int64_t *slot_mapping, int64_t num_tokens, int num_heads,
                                int head_size, int block_size, int64_t num_blocks,
                                int64_t key_stride_elems, int64_t value_stride_elems, int src_dtype,
                                int cache_elem_bytes, const float *k_scale, const float *v_scale,
                                emm_stream_t stream) {
  return append_paged(&key, &value, &key_cache, &value_cache, 1, slot_mapping, num_tokens, num_heads,
                      head_size, block_size, num_blocks, key_stride_elems, value_stride_elems, src_dtype,
                      cache_elem_bytes, k_scale, v_scale, as_stream(stream), "emm_reshape_and_cache_paged");
}

int emm_reshape_and_cache_paged_layers(const void *const *key_ptrs, const void *const *value_ptrs,
                                       void *const *key_cache_ptrs, void *const *value_cache_ptrs,
                                       int num_layers, const int64_t *slot_mapping, int64_t num_tokens,
                                       int num_heads, int head_size, int block_size, int64_t num_blocks,
                                       int64_t key_stride_elems, int64_t value_stride_elems,
                                       int src_dtype, int cache_elem_bytes, const float *k_scales,
                                       const float *v_scales, emm_stream_t stream) {
  return append_paged(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers, slot_mapping,
                      num_tokens, num_heads, head_size, block_size, num_blocks, key_stride_elems,
                      value_stride_elems, src_dtype, cache_elem_bytes, k_scales, v_scales, as_stream(stream),
                      "emm_reshape_and_cache_paged_layers");
}

int emm_concat_rows(const void *const *srcs, const int64_t *nbytes, int n, void *dst,
                    int64_t dst_offset_bytes, emm_stream_t stream) {
  const char *what = "emm_concat_rows";
  if (n < 0 || n > EMM_MAX_SEGMENTS)
    return fail(EMM_EINVAL, "%s: n=%d outside [0, %d]", what, n, EMM_MAX_SEGMENTS);
  if (n == 0) return EMM_OK;
  if (!srcs || !nbytes || !dst || dst_offset_bytes < 0)
    return fail(EMM_EINVAL, "%s: null pointer / negative offset", what);
  ConcatParams p;
  memset(&p, 0, sizeof(p));
  int al = common_align(16, (const char *)dst + dst_offset_bytes);
  int64_t off = dst_offset_bytes;
  int m = 0;
  for (int i = 0; i < n; ++i) {
    if (nbytes[i] < 0) return fail(EMM_EINVAL, "%s: nbytes[%d] negative", what, i);
    if (nbytes[i] == 0) continue;
    if (!srcs[i]) return fail(EMM_EINVAL, "%s: srcs[%d] is null", what, i);
    p.src[m] = (const char *)srcs[i];
    p.dst_off[m] = off;
    p.nbytes[m] = nbytes[i];
    al = common_align(al, srcs[i]);
    while (al > 1 && (off % al || nbytes[i] % al)) al >>= 1;
    off += nbytes[i];
    ++m;
  }
  if (m == 0) return EMM_OK;
  if (al == 8) al = 4;
  // 16-byte lanes: one vector per lane (4 KiB tiles); narrower lanes: four
  const int unroll = al == 16 ? 1 : 4;
  const int64_t tile = (int64_t)unroll * kThreads * al;
  uint64_t tiles = 0;
  for (int i = 0; i < EMM_MAX_SEGMENTS; ++i) p.tile_start[i] = 0xffffffffu;
  for (int i = 0; i < m; ++i) {
    p.tile_start[i] = (uint32_t)tiles;
    tiles += (uint64_t)((p.nbytes[i] + tile - 1) / tile);
    if (tiles > 0x7fffffffULL) return fail(EMM_EINVAL, "%s: grid too large", what);
  }
  for (int g = 0; g < kSegGroups; ++g) p.group_start[g] = p.tile_start[g * kSegGroup];
  p.dst = (char *)dst;
  dim3 grid((uint32_t)tiles);
  hipStream_t s = as_stream(stream);
  switch (al) {
  case 16: emm_concat_rows_kernel<u32x4, 1><<<grid, kThreads, 0, s>>>(p); break;
  case 4: emm_concat_rows_kernel<uint32_t, 4><<<grid, kThreads, 0, s>>>(p); break;
  case 2: emm_concat_rows_kernel<uint16_t, 4><<<grid, kThreads, 0, s>>>(p); break;
  default: emm_concat_rows_kernel<uint8_t, 4><<<grid, kThreads, 0, s>>>(p); break;
  }
  return check_launch(what);
}

} // extern "C"

// ============================================================================
// Benchmark / test hooks — compiled only with -DEMM_BENCH_HOOKS into
// libemm_kv_hooks.so, never into the product library (csrc/emm_kv_hooks.h)
// ============================================================================
#ifdef EMM_BENCH_HOOKS
#include "emm_kv_hooks.h"

namespace {

// Memory-system yardsticks with the geometry of pack / unpack: grid (tiles per chunk, n, planes),
// one 16-byte vector per lane. READ kinds fold what they load into a value that is (practically)
// never equal to the magic word, so the loads cannot be dropped and nothing is written.
template <int KIND>
__global__ __launch_bounds__(kThreads) void emm_probe_kernel(const int64_t *__restrict__ idx, char *lin,
                                                            int64_t lin_plane_stride, int64_t chunk, uint32_t nb,
                                                            uint32_t *sink, const PlaneTables<1> tables) {
  const uint32_t pl = blockIdx.z, j = blockIdx.y;
  const int64_t tile_off = (int64_t)blockIdx.x * (kThreads * 16) + threadIdx.x * 16;
  if (tile_off >= chunk) return;
  char *p;
  if constexpr (KIND == EMM_PROBE_GATHER_READ || KIND == EMM_PROBE_SCATTER_WRITE) {
    int64_t b = idx[j];
    char *plane = tables.t[0].base[pl];
    asm volatile("" : "+s"(b), "+s"(plane) : : "memory");
    if ((uint64_t)b >= (uint64_t)nb) return;
    p = plane + b * chunk + tile_off;
  } else if constexpr (KIND == EMM_PROBE_GATHER_READ_COMPUTED_IDS || KIND == EMM_PROBE_PACK_COMPUTED_IDS ||
                       KIND == EMM_PROBE_PACK || KIND == EMM_PROBE_PACK_NOTHING_FETCHED) {
    // pack with the id taken from the table, or computed (a multiplicative hash of j into [0, nb): no memory
    // round trip before the data can be requested); gathered read alone with the computed id; and the pack
    // with the plane base computed as well (planes evenly spaced from the first, whose pointer arrives
    // preloaded with the leading arguments): no scalar load at all in front of the data
    int64_t b = KIND == EMM_PROBE_PACK ? idx[j] : (int64_t)(((uint64_t)(j * 2654435761u) * nb) >> 32);
    char *plane = KIND == EMM_PROBE_PACK_NOTHING_FETCHED ? tables.t[0].base[0] + (int64_t)pl * nb * chunk
                                                         : tables.t[0].base[pl];
    asm volatile("" : "+s"(b), "+s"(plane) : : "memory");
    if ((uint64_t)b >= (uint64_t)nb) return;
    const u32x4 v = ld_stream<u32x4, 1>(plane + b * chunk + tile_off);
    if constexpr (KIND == EMM_PROBE_GATHER_READ_COMPUTED_IDS) {
      if ((v[0] ^ v[1] ^ v[2] ^ v[3]) == 0x9e3779b9u && sink) sink[threadIdx.x] = v[0];
    } else {
      st_stream<u32x4, 1>(lin + (int64_t)pl * lin_plane_stride + (int64_t)j * chunk + tile_off, v);
    }
    return;
  } else {
    p = lin + (int64_t)pl * lin_plane_stride + (int64_t)j * chunk + tile_off;
  }
  if constexpr (KIND == EMM_PROBE_SEQ_READ || KIND == EMM_PROBE_GATHER_READ) {
    const u32x4 v = ld_stream<u32x4, 1>(p);
    if ((v[0] ^ v[1] ^ v[2] ^ v[3]) == 0x9e3779b9u && sink) sink[threadIdx.x] = v[0];
  } else {
    st_stream<u32x4, 1>(p, u32x4{j, pl, 2u, 3u});
  }
}

// Other shapes of the pack kernel, kept so that the choice of the product's shape (one 16-byte load and one 16-byte
// store per lane, a 4 KiB tile per 256-thread workgroup) can be re-measured: same gather, same transfer buffer, same
// store policy; grid (pieces per chunk, blocks, planes). The chunk must be a multiple of the variant's piece.
//   U2         a workgroup moves two neighbouring tiles (8 KiB): both loads of a lane in flight before its first store
//   CHUNK      a workgroup moves four tiles (16 KiB, a whole Qwen2-7B chunk): four loads in flight, then four stores
//   LDS_1W     one-wave workgroups; the wave requests 4 x 1 KiB straight into LDS (global_load_lds_dwordx4: no data
//              registers, the loads never follow a store of the same wave), waits once, reads the LDS and stores
//   LDS_4W     the same with four waves per workgroup (16 KiB per workgroup)
//   LDS_8K     one-wave workgroups, 8 x 1 KiB per wave in flight
//   SPLIT      loader and storer waves: waves 0-1 only load (each 4 x 1 KiB per step, straight into LDS), waves 2-3
//              only store what the loaders fetched in the previous step (double buffer, one block barrier per step;
//              a workgroup walks kSplitSteps pieces of 8 KiB); a storer never waits for a load of its own and a
//              loader never for a write acknowledgement
constexpr int kSplitSteps = 8;
template <int VAR>
__global__ __launch_bounds__(VAR == EMM_PACK_VARIANT_LDS_1W || VAR == EMM_PACK_VARIANT_LDS_8K ? 64 : 256)
void emm_pack_variant_kernel(const int64_t *__restrict__ idx, char *lin, int64_t lin_plane_stride, int64_t chunk,
                             uint32_t nb, uint32_t n, const PlaneTables<1> tables) {
  typedef __attribute__((address_space(3))) void lds_void;
  const uint32_t pl = blockIdx.z, j = blockIdx.y, tid = threadIdx.x;
  if constexpr (VAR == EMM_PACK_VARIANT_SPLIT) {
    // grid x = groups of kSplitSteps pieces of 8 KiB along (block, offset in chunk) of this plane; y unused
    __shared__ __attribute__((aligned(16))) char buf[2][8192];
    const uint32_t wave = tid >> 6, lane = tid & 63;
    const uint64_t pieces_per_chunk = (uint64_t)chunk / 8192;
    const uint64_t first = (uint64_t)blockIdx.x * kSplitSteps, total = (uint64_t)n * pieces_per_chunk;
    char *plane = tables.t[0].base[pl];
    for (int step = 0; step <= kSplitSteps; ++step) {
      const uint64_t p = first + step;
      if (wave < 2) { // loaders: piece `p` into buffer step & 1
        if (step < kSplitSteps && p < total) {
          const uint64_t jb = p / pieces_per_chunk, part = p - jb * pieces_per_chunk;
          const int64_t b = idx[jb];
          if ((uint64_t)b < (uint64_t)nb) {
            const char *src = plane + b * chunk + part * 8192 + wave * 4096 + lane * 16;
#pragma unroll
            for (int i = 0; i < 4; ++i)
              __builtin_amdgcn_global_load_lds((const EMM_GLOBAL void *)(src + i * 1024),
                                               (lds_void *)(buf[step & 1] + wave * 4096 + i * 1024), 16, 0, 0);
          }
          __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): the piece is in LDS before the barrier
        }
      } else if (step > 0 && p - 1 < total) { // storers: the piece of the previous step
        const uint64_t q = p - 1, jb = q / pieces_per_chunk, part = q - jb * pieces_per_chunk;
        if ((uint64_t)idx[jb] < (uint64_t)nb) {
          char *dst = lin + (int64_t)pl * lin_plane_stride + (int64_t)jb * chunk + part * 8192 + (wave - 2) * 4096 + lane * 16;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            st_stream<u32x4, 1>(dst + i * 1024,
                                *reinterpret_cast<const u32x4 *>(buf[(step - 1) & 1] + (wave - 2) * 4096 + i * 1024 + lane * 16));
        }
      }
      __syncthreads(); // every wave reaches every barrier: the loop bounds are the same for all
    }
    return;
  } else {
    int64_t b = idx[j];
    char *plane = tables.t[0].base[pl];
    asm volatile("" : "+s"(b), "+s"(plane) : : "memory");
    if ((uint64_t)b >= (uint64_t)nb) return;
    const char *src = plane + b * chunk;
    char *dst = lin + (int64_t)pl * lin_plane_stride + (int64_t)j * chunk;
    if constexpr (VAR == EMM_PACK_VARIANT_U2 || VAR == EMM_PACK_VARIANT_CHUNK) {
      constexpr int U = VAR == EMM_PACK_VARIANT_U2 ? 2 : 4;
      const int64_t off = (int64_t)blockIdx.x * (U * 4096) + tid * 16;
      u32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = ld_stream<u32x4, 1>(src + off + u * 4096);
#pragma unroll
      for (int u = 0; u < U; ++u) st_stream<u32x4, 1>(dst + off + u * 4096, v[u]);
    } else {
      constexpr int K = VAR == EMM_PACK_VARIANT_LDS_8K ? 8 : 4;               // 1 KiB loads per wave
      constexpr int W = VAR == EMM_PACK_VARIANT_LDS_4W ? 4 : 1;               // waves per workgroup
      __shared__ __attribute__((aligned(16))) char tile[W * K * 1024];
      const uint32_t wave = tid >> 6, lane = tid & 63;
      const int64_t off = ((int64_t)blockIdx.x * W + wave) * (K * 1024) + lane * 16;
#pragma unroll
      for (int i = 0; i < K; ++i)
        __builtin_amdgcn_global_load_lds((const EMM_GLOBAL void *)(src + off + i * 1024),
                                         (lds_void *)(tile + (wave * K + i) * 1024), 16, 0, 0);
      __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0)
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
#pragma unroll
      for (int i = 0; i < K; ++i)
        st_stream<u32x4, 1>(dst + off + i * 1024, *reinterpret_cast<const u32x4 *>(tile + (wave * K + i) * 1024 + lane * 16));
    }
  }
}

// A kernel that does nothing: a chain of these measures what a dependent launch costs by itself.
__global__ void emm_empty_kernel() {}

// The fast quotient against the division for one exponent pair and a range of scale significands:
// thread = one scale significand, loop over all 2^10 x significands (the 11 significant bits of an
// f16; bf16 values are the subset with 3 more trailing zeros) and both signs.
// counters[0] raw fp32 quotients that differ from RN(x / s) (counted where the division's result is
// a normal number), [1] differing e4m3fn bytes (torch mode), [2] differing bytes (saturating mode),
// [3] pairs checked, [4] (x bits << 32 | s bits) of one differing pair.
__global__ __launch_bounds__(kThreads) void emm_quotient_sweep_kernel(int x_exp, int s_exp, uint32_t s_begin,
                                                                      uint32_t s_end,
                                                                      unsigned long long *counters) {
  const uint32_t ms = s_begin + blockIdx.x * kThreads + threadIdx.x;
  if (ms >= s_end) return;
  const uint32_t sbits = ((uint32_t)(s_exp + 127) << 23) | ms;
  const float s = __uint_as_float(sbits);
  const Divisor d = make_divisor(s, true);
  unsigned long long bad_raw = 0, bad_byte = 0, bad_sat = 0, bad_pair = 0;
  for (uint32_t mx = 0; mx < 2048; ++mx) {
    const uint32_t xbits = ((mx & 1024u) << 21) | ((uint32_t)(x_exp + 127) << 23) | ((mx & 1023u) << 13);
    const float x = __uint_as_float(xbits);
    const float ref = x / s;
    const float fast = d.exact_fast ? divide_fast_raw(x, d) : ref;
    const uint32_t rb = __float_as_uint(ref), fb = __float_as_uint(fast);
    const bool normal = (rb & 0x7f800000u) != 0 && (rb & 0x7f800000u) != 0x7f800000u;
    if (normal && rb != fb) {
      ++bad_raw;
      bad_pair = ((unsigned long long)xbits << 32) | sbits;
    }
    const float f0 = d.exact_fast ? divide_fast<false>(x, d) : divide_ieee<false>(x, s);
    const float f1 = d.exact_fast ? divide_fast<true>(x, d) : divide_ieee<true>(x, s);
    const float r0 = divide_ieee<false>(x, s), r1 = divide_ieee<true>(x, s);
    const int b0 = __builtin_amdgcn_cvt_pk_fp8_f32(f0, f0, 0, false) & 0xff;
    const int c0 = __builtin_amdgcn_cvt_pk_fp8_f32(r0, r0, 0, false) & 0xff;
    const int b1 = __builtin_amdgcn_cvt_pk_fp8_f32(f1, f1, 0, false) & 0xff;
    const int c1 = __builtin_amdgcn_cvt_pk_fp8_f32(r1, r1, 0, false) & 0xff;
    if (b0 != c0) {
      ++bad_byte;
      bad_pair = ((unsigned long long)xbits << 32) | sbits;
    }
    if (b1 != c1) ++bad_sat;
  }
  if (bad_raw) atomicAdd(&counters[0], bad_raw);
  if (bad_byte) atomicAdd(&counters[1], bad_byte);
  if (bad_sat) atomicAdd(&counters[2], bad_sat);
  atomicAdd(&counters[3], 2048ull);
  if (bad_pair) atomicMax(&counters[4], bad_pair);
}

} // namespace

extern "C" {

int emm_hook_set_move_variant(int variant) {
  const int old = g_move_variant;
  g_move_variant = variant & 0x7fffff00;
  return old;
}

int emm_hook_probe(int kind, void *const *layer_ptrs, int num_layers, int num_kv, int64_t num_blocks,
                   int64_t chunk_bytes, const int64_t *block_idx, int64_t n, void *linear, uint32_t *sink,
                   emm_stream_t stream) {
  const char *what = "emm_hook_probe";
  if (kind < 0 || kind > EMM_PROBE_PACK_NOTHING_FETCHED) return fail(EMM_EINVAL, "%s: unknown kind %d", what, kind);
  const bool pool = kind >= EMM_PROBE_GATHER_READ; // every kind but the two sequential ones walks the pool's planes
  const bool linear_too = kind == EMM_PROBE_PACK || kind == EMM_PROBE_PACK_COMPUTED_IDS || kind == EMM_PROBE_PACK_NOTHING_FETCHED;
  if (num_layers <= 0 || num_layers > EMM_MAX_LAYERS || num_kv <= 0 || n <= 0 || n > kMaxGridY || chunk_bytes <= 0 ||
      chunk_bytes % 16)
    return fail(EMM_EINVAL, "%s: bad geometry", what);
  if (pool && (!layer_ptrs || !block_idx || num_blocks <= 0 || num_blocks > 0x7fffffffLL))
    return fail(EMM_EINVAL, "%s: pool kinds need layer_ptrs, block_idx and num_blocks", what);
  if ((!pool || linear_too) && (!linear || !aligned(linear, 16)))
    return fail(EMM_EINVAL, "%s: linear kinds need a 16-byte aligned buffer", what);
  PlaneTables<1> t;
  memset(&t, 0, sizeof(t));
  const int planes = num_layers * num_kv;
  if (pool)
    for (int i = 0; i < planes; ++i) {
      if (!layer_ptrs[i / num_kv] || !aligned(layer_ptrs[i / num_kv], 16)) return fail(EMM_EINVAL, "%s: bad layer pointer", what);
      t.t[0].base[i] = (char *)layer_ptrs[i / num_kv] + (int64_t)(i % num_kv) * num_blocks * chunk_bytes;
    }
  if (kind == EMM_PROBE_PACK_NOTHING_FETCHED)
    for (int i = 0; i < planes; ++i)
      if (t.t[0].base[i] != t.t[0].base[0] + (int64_t)i * num_blocks * chunk_bytes)
        return fail(EMM_EINVAL, "%s: this kind needs a pool whose planes are evenly spaced (one allocation)", what);
  const dim3 grid((uint32_t)((chunk_bytes + kThreads * 16 - 1) / (kThreads * 16)), (uint32_t)n, (uint32_t)planes);
  hipStream_t s = as_stream(stream);
  char *lin = (char *)linear;
  const int64_t stride = n * chunk_bytes;
  switch (kind) {
  case EMM_PROBE_SEQ_READ: emm_probe_kernel<EMM_PROBE_SEQ_READ><<<grid, kThreads, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, sink, t); break;
  case EMM_PROBE_SEQ_WRITE: emm_probe_kernel<EMM_PROBE_SEQ_WRITE><<<grid, kThreads, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, sink, t); break;
  case EMM_PROBE_GATHER_READ: emm_probe_kernel<EMM_PROBE_GATHER_READ><<<grid, kThreads, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, sink, t); break;
  case EMM_PROBE_SCATTER_WRITE: emm_probe_kernel<EMM_PROBE_SCATTER_WRITE><<<grid, kThreads, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, sink, t); break;
  case EMM_PROBE_GATHER_READ_COMPUTED_IDS: emm_probe_kernel<EMM_PROBE_GATHER_READ_COMPUTED_IDS><<<grid, kThreads, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, sink, t); break;
  case EMM_PROBE_PACK_COMPUTED_IDS: emm_probe_kernel<EMM_PROBE_PACK_COMPUTED_IDS><<<grid, kThreads, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, sink, t); break;
  case EMM_PROBE_PACK: emm_probe_kernel<EMM_PROBE_PACK><<<grid, kThreads, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, sink, t); break;
  case EMM_PROBE_PACK_NOTHING_FETCHED: emm_probe_kernel<EMM_PROBE_PACK_NOTHING_FETCHED><<<grid, kThreads, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, sink, t); break;
  default: return fail(EMM_EINVAL, "%s: unknown kind %d", what, kind);
  }
  return check_launch(what);
}

int emm_hook_pack_variant(int variant, const void *const *layer_ptrs, int num_layers, int num_kv, int64_t num_blocks,
                          int64_t chunk_bytes, const int64_t *block_idx, int64_t n, void *packed, emm_stream_t stream) {
  const char *what = "emm_hook_pack_variant";
  if (variant < EMM_PACK_VARIANT_U2 || variant > EMM_PACK_VARIANT_SPLIT) return fail(EMM_EINVAL, "%s: unknown variant %d", what, variant);
  if (num_layers <= 0 || num_layers > EMM_MAX_LAYERS || num_kv <= 0 || n <= 0 || n > kMaxGridY || num_blocks <= 0 ||
      num_blocks > 0x7fffffffLL || !layer_ptrs || !block_idx || !packed || !aligned(packed, 16))
    return fail(EMM_EINVAL, "%s: bad geometry / null pointer", what);
  const int64_t piece = variant == EMM_PACK_VARIANT_U2 || variant == EMM_PACK_VARIANT_LDS_8K || variant == EMM_PACK_VARIANT_SPLIT ? 8192
                        : variant == EMM_PACK_VARIANT_LDS_1W ? 4096 : 16384;
  if (chunk_bytes <= 0 || chunk_bytes % piece) return fail(EMM_EINVAL, "%s: chunk must be a multiple of %lld bytes", what, (long long)piece);
  PlaneTables<1> t;
  memset(&t, 0, sizeof(t));
  const int planes = num_layers * num_kv;
  for (int i = 0; i < planes; ++i) {
    if (!layer_ptrs[i / num_kv] || !aligned(layer_ptrs[i / num_kv], 16)) return fail(EMM_EINVAL, "%s: bad layer pointer", what);
    t.t[0].base[i] = (char *)layer_ptrs[i / num_kv] + (int64_t)(i % num_kv) * num_blocks * chunk_bytes;
  }
  hipStream_t s = as_stream(stream);
  char *lin = (char *)packed;
  const int64_t stride = n * chunk_bytes;
  const dim3 grid((uint32_t)(chunk_bytes / piece), (uint32_t)n, (uint32_t)planes);
#define EMM_PV(V_, T_) emm_pack_variant_kernel<V_><<<grid, T_, 0, s>>>(block_idx, lin, stride, chunk_bytes, (uint32_t)num_blocks, (uint32_t)n, t)
  switch (variant) {
  case EMM_PACK_VARIANT_U2: EMM_PV(EMM_PACK_VARIANT_U2, 256); break;
  case EMM_PACK_VARIANT_CHUNK: EMM_PV(EMM_PACK_VARIANT_CHUNK, 256); break;
  case EMM_PACK_VARIANT_LDS_1W: EMM_PV(EMM_PACK_VARIANT_LDS_1W, 64); break;
  case EMM_PACK_VARIANT_LDS_4W: EMM_PV(EMM_PACK_VARIANT_LDS_4W, 256); break;
  case EMM_PACK_VARIANT_LDS_8K: EMM_PV(EMM_PACK_VARIANT_LDS_8K, 64); break;
  default: {
    const int64_t pieces = n * (chunk_bytes / 8192);
    const dim3 sgrid((uint32_t)((pieces + kSplitSteps - 1) / kSplitSteps), 1, (uint32_t)planes);
    emm_pack_variant_kernel<EMM_PACK_VARIANT_SPLIT><<<sgrid, 256, 0, s>>>(block_idx, lin, stride, chunk_bytes,
                                                                          (uint32_t)num_blocks, (uint32_t)n, t);
  }
  }
#undef EMM_PV
  return check_launch(what);
}

int emm_hook_empty_launch(emm_stream_t stream) {
  emm_empty_kernel<<<1, 64, 0, as_stream(stream)>>>();
  return check_launch("emm_hook_empty_launch");
}

int emm_hook_fp8_quotient_sweep(int x_exp, int s_exp, uint32_t s_begin, uint32_t s_end, uint64_t *counters,
                                emm_stream_t stream) {
  const char *what = "emm_hook_fp8_quotient_sweep";
  if (x_exp < -126 || x_exp > 127 || s_exp < -126 || s_exp > 127) return fail(EMM_EINVAL, "%s: exponent out of range", what);
  if (s_begin >= s_end || s_end > (1u << 23)) return fail(EMM_EINVAL, "%s: bad significand range", what);
  if (!counters) return fail(EMM_EINVAL, "%s: null counters", what);
  const uint32_t blocks = (s_end - s_begin + kThreads - 1) / kThreads;
  emm_quotient_sweep_kernel<<<blocks, kThreads, 0, as_stream(stream)>>>(x_exp, s_exp, s_begin, s_end,
                                                                        (unsigned long long *)counters);
  return check_launch(what);
}

} // extern "C"
#endif // EMM_BENCH_HOOKS
