// kvmove.hip -- KV-block migration and swap for MI355X (gfx950, wave64).
//
// The whole path is byte movement, so there is no MFMA here.  One piece of tile-copy code
// serves migration (gather by block-index tables + re-slice of layers/heads between the
// context instance's TP/PP layout and one decoding rank), the kernel flavour of swap, and
// the plain calibration copy, in three launch forms: kvm_copy_kernel (any shape),
// kvm_copy_simple_kernel (layouts that agree) and kvm_walk_kernel (link-bound).  The
// metadata (segment table and block-index pairs) travels in the kernel-argument segment,
// so every workgroup picks it up with scalar loads into SGPRs and no device-side table,
// staging copy or allocation exists anywhere on the path.
//
// Reference call sites this stands behind: distserve/worker.py:133-134 (handles),
// :239-246 (registration), :250-267 (migrate_blocks), :303-311 (swap).
#include "kvmove.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstddef>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <shared_mutex>
#include <string>
#include <tuple>
#include <vector>
#include <time.h>
#include <unistd.h>

namespace {

// ------------------------------------------------------------------ kernel argument

constexpr int kMaxSegs = 8;          // source segments per launch
constexpr int kMaxIdx = 432;         // block-index pairs per launch as two int32 (keeps the argument <= 4 KiB)
constexpr int kMaxIdxPacked = 864;   // ... as two uint16 in one word, when both pools have at most 65536 blocks

// One rectangle of the decoding rank's block that a single context rank supplies:
// n_rows runs of run_bytes, one per overlapping layer.
struct Seg {
    const char *src_k;         // context pool base + offset of the rectangle inside a block
    const char *src_v;
    uint64_t src_block_stride; // bytes per source block
    uint32_t src_row_stride;   // bytes between consecutive layers in the source block
    uint32_t dst_row_stride;   // ... in the destination block
    uint32_t dst_off;          // offset of the rectangle inside a destination block
    uint32_t run_bytes;        // contiguous bytes per row
    uint32_t n_rows;
    uint32_t rows_per_tile;    // >1 only when a whole row is smaller than a tile
    uint32_t pieces_per_row;   // >1 only when a row is larger than a tile
    uint32_t piece_bytes;
    uint32_t pieces_magic;     // tile / pieces_per_row without a divider: see fast_div
    uint32_t pieces_shifts;
};
static_assert(sizeof(Seg) == 64 && offsetof(Seg, src_row_stride) == 24 && offsetof(Seg, pieces_shifts) == 60,
              "Seg layout: the kernel reads it as 16 dwords");

struct IdxPair {
    int32_t ctx;  // block in the context pools
    int32_t dec;  // block in the decoding pool
};

// The first 64 bytes are everything a workgroup needs before it knows its segment; they
// come in with one 16-dword scalar load.
struct MigrateArgs {
    char *dst_k;
    char *dst_v;
    uint64_t dst_block_stride;
    uint32_t nseg;
    uint32_t nidx;
    uint32_t tile_end[kMaxSegs];  // exclusive prefix sums of tiles per segment; UINT32_MAX past the last
    // second header record: how a workgroup id becomes (block, tile)
    uint32_t tiles_per_block;     // T: tiles of one block of one pool kind
    uint32_t tiles_magic, tiles_shifts;
    uint32_t chunk_tiles;         // C: consecutive work items one XCD takes at a time; 0 = ids in order
    uint32_t chunk_magic, chunk_shifts;
    uint32_t work;                // W = T * nidx work items per pool kind
    uint32_t work_padded;         // grid.x / 2: W rounded up so that every XCD gets whole chunks
    Seg seg[kMaxSegs];
    union {
        IdxPair idx[kMaxIdx];
        uint32_t packed[kMaxIdxPacked];   // context block | decoding block << 16
    };
};
static_assert(sizeof(MigrateArgs) <= 4096, "kernel argument must stay within 4 KiB");

// ------------------------------------------------------------------------- device

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint64_t u64_of(uint32_t lo, uint32_t hi) { return ((uint64_t)hi << 32) | lo; }

// Kernel flavour bits (template parameter FLAGS).
constexpr int kNtLoad = 1;      // nontemporal loads
constexpr int kNtStore = 2;     // nontemporal stores
constexpr int kWaveContig = 4;  // a wave's UNROLL vectors are adjacent in memory (else one pass apart)

// Pool memory is addressed through global-address-space pointers, so that lanes issue
// global_load/global_store (not flat ones) although the addresses are built from integers.
#define KVM_GLOBAL __attribute__((address_space(1)))
typedef KVM_GLOBAL char gchar;

template <int FLAGS, typename V>
__device__ __forceinline__ V ld(const KVM_GLOBAL V *p)
{
    if constexpr ((FLAGS & kNtLoad) != 0) return __builtin_nontemporal_load(p);
    else return *p;
}

// Nontemporal stores of 16-byte vectors carry "sc1 nt" (streaming, written through beyond
// the XCD's L2), which only inline assembly can express; beside nontemporal loads it
// measured 0.5-2 % faster than "nt" alone.  Narrower vectors use the compiler's "nt".
// The s_nop belongs to the store: a store of more than 8 bytes reads its data registers
// for two more cycles, and the compiler, which cannot see that this text is such a store,
// may otherwise reuse them at once.
template <int FLAGS, typename V>
__device__ __forceinline__ void st(KVM_GLOBAL V *p, V v)
{
    if constexpr ((FLAGS & kNtStore) != 0) {
        if constexpr (sizeof(V) == 16) {
            asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
        } else {
            __builtin_nontemporal_store(v, p);
        }
    } else {
        *p = v;
    }
}

// Byte offset, inside one step of THREADS*UNROLL vectors, of this lane's u-th vector.
template <typename V, int THREADS, int UNROLL, int FLAGS>
__device__ __forceinline__ uint32_t vec_off(int u)
{
    constexpr uint32_t kVec = (uint32_t)sizeof(V);
    if constexpr ((FLAGS & kWaveContig) != 0) {
        const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        return (wave * UNROLL + u) * (64 * kVec) + lane * kVec;
    } else {
        return (u * THREADS + threadIdx.x) * kVec;
    }
}

// One contiguous run of `len` bytes (a multiple of sizeof(V)) by the whole workgroup:
// UNROLL independent loads per lane are issued before the first store.  With
// len <= THREADS * UNROLL * sizeof(V) the workgroup is "one shot": all loads, all stores,
// end -- no wave ever waits for its own stores before it can load again.
template <typename V, int THREADS, int UNROLL, int FLAGS>
__device__ __forceinline__ void copy_run(gchar *dst, const gchar *src, uint32_t len)
{
    constexpr uint32_t kStep = THREADS * UNROLL * (uint32_t)sizeof(V);
    uint32_t off = 0;
    for (; off + kStep <= len; off += kStep) {
        V r[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            r[u] = ld<FLAGS>(reinterpret_cast<const KVM_GLOBAL V *>(src + off + vec_off<V, THREADS, UNROLL, FLAGS>(u)));
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            st<FLAGS>(reinterpret_cast<KVM_GLOBAL V *>(dst + off + vec_off<V, THREADS, UNROLL, FLAGS>(u)), r[u]);
    }
    if (off < len) {
        V r[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t o = off + vec_off<V, THREADS, UNROLL, FLAGS>(u);
            if (o < len) r[u] = ld<FLAGS>(reinterpret_cast<const KVM_GLOBAL V *>(src + o));
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t o = off + vec_off<V, THREADS, UNROLL, FLAGS>(u);
            if (o < len) st<FLAGS>(reinterpret_cast<KVM_GLOBAL V *>(dst + o), r[u]);
        }
    }
}

// `nrows` runs of `len` bytes each, `sstride` / `dstride` apart: the UNROLL loads in
// flight span row boundaries, so short rows still keep several loads outstanding.
// The (row, pass-in-row) counters are wave-uniform and advance in SGPRs.
template <typename V, int THREADS, int UNROLL, int FLAGS>
__device__ __forceinline__ void copy_rows(gchar *dst, const gchar *src, uint32_t nrows, uint32_t len,
                                          uint32_t sstride, uint32_t dstride)
{
    constexpr uint32_t kPass = THREADS * (uint32_t)sizeof(V);
    const uint32_t lane_off = threadIdx.x * (uint32_t)sizeof(V);
    const uint32_t passes_per_row = (len + kPass - 1) / kPass;
    const uint32_t total_passes = nrows * passes_per_row;
    uint32_t row = 0, pc = 0;
    for (uint32_t q = 0; q < total_passes; q += UNROLL) {
        V r[UNROLL];
        uint32_t soff[UNROLL], doff[UNROLL];
        bool ok[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t col = pc * kPass + lane_off;
            ok[u] = (row < nrows) && (col < len);
            soff[u] = row * sstride + col;
            doff[u] = row * dstride + col;
            if (++pc == passes_per_row) { pc = 0; ++row; }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            if (ok[u]) r[u] = ld<FLAGS>(reinterpret_cast<const KVM_GLOBAL V *>(src + soff[u]));
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            if (ok[u]) st<FLAGS>(reinterpret_cast<KVM_GLOBAL V *>(dst + doff[u]), r[u]);
    }
}

// n / d for a divisor fixed on the host: magic and shifts from make_magic (round-up method
// with a 33-bit multiplier folded into an add and two shifts; exact for every 32-bit n).
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t magic, uint32_t shifts)
{
    const uint32_t t = __umulhi(magic, n);
    return (t + ((n - t) >> (shifts & 0xffu))) >> (shifts >> 8);
}

// The index pair of one block, from either form of the table.
template <bool PACKED>
__device__ __forceinline__ void load_pair(const MigrateArgs &a, uint32_t pair, uint32_t &ctx, uint32_t &dec)
{
    if constexpr (PACKED) {
        const uint32_t p = a.packed[pair];
        ctx = p & 0xffffu;
        dec = p >> 16;
    } else {
        const IdxPair ix = a.idx[pair];
        ctx = (uint32_t)ix.ctx;
        dec = (uint32_t)ix.dec;
    }
}

// One tile of one block of one pool kind.  Everything up to the lane offset is
// wave-uniform and lives in SGPRs.  The scalar loads are arranged for a short dependent
// chain, because a workgroup here lives for little more than one memory round trip: the
// header (with every segment's tile range) and the block-index pair are independent
// loads, the segment's fields are the one dependent round after them.
template <typename V, int THREADS, int UNROLL, int FLAGS, bool PACKED>
__device__ __forceinline__ void do_tile(const MigrateArgs &a, const u32x16 h, uint32_t tile, uint32_t pair, bool is_v)
{
    // `h` is the first header record (64 bytes, one 16-dword scalar load by the caller); the
    // segment is a second 64-byte record fetched whole, so that the dependent chain is
    // {header records} -> {index pair, segment} -> addresses.
    static_assert(offsetof(MigrateArgs, tile_end) == 32 && offsetof(MigrateArgs, tiles_per_block) == 64 &&
                      offsetof(MigrateArgs, seg) == 96, "header layout");
    uint32_t ctx, dec;
    load_pair<PACKED>(a, pair, ctx, dec);
    uint32_t s = 0, tile_begin = 0;
#pragma unroll
    for (int j = 0; j < kMaxSegs - 1; ++j) {
        if (tile >= h[8 + j]) {
            s = j + 1;
            tile_begin = h[8 + j];
        }
    }
    tile -= tile_begin;
    const u32x16 g = *reinterpret_cast<const u32x16 *>(&a.seg[s]);
    const uint64_t src_base = is_v ? u64_of(g[2], g[3]) : u64_of(g[0], g[1]);
    const uint64_t dst_base = is_v ? u64_of(h[2], h[3]) : u64_of(h[0], h[1]);
    const uint64_t src_block_stride = u64_of(g[4], g[5]), dst_block_stride = u64_of(h[4], h[5]);
    const uint32_t src_row_stride = g[6], dst_row_stride = g[7], dst_off = g[8], run_bytes = g[9];
    const uint32_t n_rows = g[10], rows_per_tile = g[11], pieces_per_row = g[12], piece_bytes = g[13];

    const gchar *src = reinterpret_cast<const gchar *>(src_base + (uint64_t)ctx * src_block_stride);
    gchar *dst = reinterpret_cast<gchar *>(dst_base + (uint64_t)dec * dst_block_stride + dst_off);

    if (rows_per_tile == 1) {
        const uint32_t row = fast_div(tile, g[14], g[15]);
        const uint32_t piece = tile - row * pieces_per_row;
        const uint32_t col_off = piece * piece_bytes;
        const uint32_t len = min(piece_bytes, run_bytes - col_off);
        copy_run<V, THREADS, UNROLL, FLAGS>(dst + (uint64_t)row * dst_row_stride + col_off,
                                            src + (uint64_t)row * src_row_stride + col_off, len);
    } else {
        const uint32_t row0 = tile * rows_per_tile;
        const uint32_t nrows = min(rows_per_tile, n_rows - row0);
        copy_rows<V, THREADS, UNROLL, FLAGS>(dst + (uint64_t)row0 * dst_row_stride,
                                             src + (uint64_t)row0 * src_row_stride, nrows, run_bytes,
                                             src_row_stride, dst_row_stride);
    }
}

// HBM-bound form: a 1-D grid of 2 * work_padded workgroups (K pool first, then V), one tile
// per workgroup, so that thousands of short-lived workgroups keep every channel busy.
//
// Workgroup ids are dealt round-robin to the 8 XCDs.  With ids in order, every XCD would
// touch every 8th KiB of every stream; instead id -> (xcd = id % 8, seq = id / 8) is turned
// into a work item such that each XCD walks its own contiguous chunks of `chunk_tiles`
// tiles (chunk number seq / C * 8 + xcd).  Chunks of 256 KiB and more measured 2-3 % faster
// than in-order ids, chunks of 2-64 KiB 5-10 % slower.
template <typename V, int THREADS, int UNROLL, int FLAGS, bool PACKED>
__global__ __launch_bounds__(THREADS) void kvm_copy_kernel(const MigrateArgs a)
{
    // both header records in one round of scalar loads
    const u32x16 h = *reinterpret_cast<const u32x16 *>(&a);
    const u32x8 m = *reinterpret_cast<const u32x8 *>(&a.tiles_per_block);
    const uint32_t tiles_per_block = m[0], chunk_tiles = m[3], work = m[6], work_padded = m[7];
    uint32_t id = blockIdx.x;
    const bool is_v = id >= work_padded;
    if (is_v) id -= work_padded;
    uint32_t w = id;
    if (chunk_tiles != 0) {
        const uint32_t xcd = id & 7u, seq = id >> 3;
        const uint32_t q = fast_div(seq, m[4], m[5]);
        w = (q * 8u + xcd) * chunk_tiles + (seq - q * chunk_tiles);
    }
    // Padding ids past the last chunk end here.  nidx (h[7]) is never 0; naming it in this
    // test keeps the first record's load in the same round as the second's instead of
    // behind the branch.
    if (w >= work || h[7] == 0) return;
    const uint32_t pair = fast_div(w, m[1], m[2]);
    do_tile<V, THREADS, UNROLL, FLAGS, PACKED>(a, h, w - pair * tiles_per_block, pair, is_v);
}

// The same for the plainest shape: one segment whose rows collapsed into a single run that
// is a whole number of full tiles (context and decoding layouts agree, e.g. TP1 -> TP1).
// Nothing depends on the tile's position but two multiplications, so the scalar prologue is
// one round of loads for the three records, the index pair, and a dozen SALU instructions.
template <typename V, int THREADS, int UNROLL, int FLAGS, bool PACKED>
__global__ __launch_bounds__(THREADS) void kvm_copy_simple_kernel(const MigrateArgs a)
{
    constexpr uint32_t kTile = THREADS * UNROLL * (uint32_t)sizeof(V);
    const u32x16 h = *reinterpret_cast<const u32x16 *>(&a);
    const u32x8 m = *reinterpret_cast<const u32x8 *>(&a.tiles_per_block);
    const u32x16 g = *reinterpret_cast<const u32x16 *>(&a.seg[0]);
    const uint32_t tiles_per_block = m[0], chunk_tiles = m[3], work = m[6], work_padded = m[7];
    uint32_t id = blockIdx.x;
    const bool is_v = id >= work_padded;
    if (is_v) id -= work_padded;
    uint32_t w = id;
    if (chunk_tiles != 0) {
        const uint32_t xcd = id & 7u, seq = id >> 3;
        const uint32_t q = fast_div(seq, m[4], m[5]);
        w = (q * 8u + xcd) * chunk_tiles + (seq - q * chunk_tiles);
    }
    if (w >= work || h[7] == 0 || g[10] == 0) return;   // (names h and g: see kvm_copy_kernel)
    const uint32_t pair = fast_div(w, m[1], m[2]);
    const uint32_t tile = w - pair * tiles_per_block;
    uint32_t ctx, dec;
    load_pair<PACKED>(a, pair, ctx, dec);
    const uint64_t src_base = is_v ? u64_of(g[2], g[3]) : u64_of(g[0], g[1]);
    const uint64_t dst_base = is_v ? u64_of(h[2], h[3]) : u64_of(h[0], h[1]);
    const uint64_t off = (uint64_t)tile * kTile;
    const gchar *src = reinterpret_cast<const gchar *>(src_base + (uint64_t)ctx * u64_of(g[4], g[5]) + off);
    gchar *dst = reinterpret_cast<gchar *>(dst_base + (uint64_t)dec * u64_of(h[4], h[5]) + g[8] + off);
    V r[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
        r[u] = ld<FLAGS>(reinterpret_cast<const KVM_GLOBAL V *>(src + vec_off<V, THREADS, UNROLL, FLAGS>(u)));
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
        st<FLAGS>(reinterpret_cast<KVM_GLOBAL V *>(dst + vec_off<V, THREADS, UNROLL, FLAGS>(u)), r[u]);
}

// Link-bound form: grid = (a few workgroups, 2 = {K, V}); each workgroup walks the
// (block, tile) pairs of the launch with a stride of gridDim.x.  A copy that the host link
// limits to tens of GB/s needs only a handful of workgroups in flight, and leaves the rest
// of the GPU to whatever runs beside it.
template <typename V, bool PACKED, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void kvm_walk_kernel(const MigrateArgs a, uint32_t tiles_per_block)
{
    const uint32_t total = a.nidx * tiles_per_block;
    for (uint32_t w = blockIdx.x; w < total; w += gridDim.x) {
        const uint32_t pair = w / tiles_per_block;
        do_tile<V, THREADS, UNROLL, kNtLoad | kNtStore, PACKED>(a, *reinterpret_cast<const u32x16 *>(&a),
                                                                w - pair * tiles_per_block, pair, blockIdx.y != 0);
    }
}

// --------------------------------------------------------------------------- host

thread_local std::string g_err;

int fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

#define KVM_HIP(expr)                                                                          \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess)                                                                  \
            return fail(KVM_EHIP, "%s failed: %s", #expr, hipGetErrorString(e_));              \
    } while (0)

// ---- options
//
// The library ships one flavour of the copy kernel (a single-wave workgroup that moves 1 KiB,
// nontemporal both ways: the one every sweep chose) and the options a deployment may want to
// set.  The exploration build (-DKVM_EXPLORE, used by sweeps and by the tests that show every
// flavour copies the same bytes) adds the other flavours and the knobs that select them.

std::atomic<int64_t> opt_swap_mode{3};
std::atomic<int64_t> opt_swap_wgs{16};
std::atomic<int64_t> opt_swap_wgs_in{16};
std::atomic<int64_t> opt_swap_kernel_below{1ll << 32};
std::atomic<int64_t> opt_xcd_map{1};
std::atomic<int64_t> opt_sort_pairs{1};
#ifdef KVM_EXPLORE
std::atomic<int64_t> opt_tile_bytes{0};
std::atomic<int64_t> opt_threads{64};
std::atomic<int64_t> opt_unroll{1};
std::atomic<int64_t> opt_nt_load{1};
std::atomic<int64_t> opt_nt_store{1};
std::atomic<int64_t> opt_lds_pad{0};
std::atomic<int64_t> opt_wave_contig{0};
std::atomic<int64_t> opt_simple{1};
std::atomic<int64_t> opt_max_pairs{kMaxIdxPacked};
std::atomic<int64_t> opt_packed{1};
std::atomic<int64_t> opt_swap_threads{256};
std::atomic<int64_t> opt_swap_unroll{1};
int64_t tune_tile_bytes() { return opt_tile_bytes.load(); }
int64_t tune_lds_pad() { return opt_lds_pad.load(); }
bool tune_simple() { return opt_simple.load() != 0; }
int64_t tune_max_pairs() { return opt_max_pairs.load(); }
bool tune_packed() { return opt_packed.load() != 0; }
#else
constexpr int64_t tune_tile_bytes() { return 0; }
constexpr int64_t tune_lds_pad() { return 0; }
constexpr bool tune_simple() { return true; }
constexpr int64_t tune_max_pairs() { return kMaxIdxPacked; }
constexpr bool tune_packed() { return true; }
#endif

std::atomic<int64_t> *find_opt(const char *name)
{
    if (!name) return nullptr;
    if (!strcmp(name, "swap_mode")) return &opt_swap_mode;
    if (!strcmp(name, "swap_wgs")) return &opt_swap_wgs;
    if (!strcmp(name, "swap_wgs_in")) return &opt_swap_wgs_in;
    if (!strcmp(name, "swap_kernel_below")) return &opt_swap_kernel_below;
    if (!strcmp(name, "xcd_map")) return &opt_xcd_map;
    if (!strcmp(name, "sort_pairs")) return &opt_sort_pairs;
#ifdef KVM_EXPLORE
    if (!strcmp(name, "tile_bytes")) return &opt_tile_bytes;
    if (!strcmp(name, "threads")) return &opt_threads;
    if (!strcmp(name, "unroll")) return &opt_unroll;
    if (!strcmp(name, "nt_load")) return &opt_nt_load;
    if (!strcmp(name, "nt_store")) return &opt_nt_store;
    if (!strcmp(name, "lds_pad")) return &opt_lds_pad;
    if (!strcmp(name, "wave_contig")) return &opt_wave_contig;
    if (!strcmp(name, "simple")) return &opt_simple;
    if (!strcmp(name, "max_pairs")) return &opt_max_pairs;
    if (!strcmp(name, "packed")) return &opt_packed;
    if (!strcmp(name, "swap_threads")) return &opt_swap_threads;
    if (!strcmp(name, "swap_unroll")) return &opt_swap_unroll;
#endif
    return nullptr;
}

// ---- registry of context pools, keyed by (context instance, pp_rank, tp_rank)

struct Source {
    int32_t ctx_pp_size, ctx_tp_size;
    int64_t num_layers, num_kv_heads;
    const char *k, *v;
    int64_t nbytes;
    const char *map_k, *map_v;   // local base of the other process's allocation each pool lies in, or null
};

using SourceKey = std::tuple<int64_t, int32_t, int32_t>;

// g_mu guards g_sources.  A migrate call holds it shared from the lookup of its pools until its
// last launch is enqueued, so that a mapping it reads through cannot be closed in between;
// registrations and resets take it exclusively, and only for the insert of a binding or for
// the sequence {drop bindings, wait for the device, unmap}.  g_reg_mu serialises registrations
// and resets among themselves (they may map memory and wait for the device, with g_mu free);
// g_opened is only touched under it.
std::shared_mutex g_mu;
std::mutex g_reg_mu;
std::map<SourceKey, Source> g_sources;

// Allocations of other processes that registration has mapped into this one.  One entry per
// (exporting process, allocation): hipIpcOpenMemHandle is called once however many pools lie
// in the allocation, and the mapping stays while a registered pool lies in it.
struct Opened {
    int64_t pid, nonce, remote_base, size;
    int64_t serial;      // the exporter's id of the allocation (0 = it had none to give)
    uint64_t opened_in;  // the registration call that opened it
    char *local_base;
};
std::vector<Opened> g_opened;
uint64_t g_reg_call = 0;        // counts registration calls; guarded by g_reg_mu

// Handle words (int64 each).
enum {
    kHwMagic = 0, kHwPid, kHwDevice, kHwPtr, kHwBytes, kHwAllocBase, kHwAllocSize, kHwFlags,
    kHwIpc = 8,                                  // 8 words = the 64 bytes of a hipIpcMemHandle_t
    kHwNonce = 16,
    kHwCheck = 17,
};
static_assert(sizeof(hipIpcMemHandle_t) == 64 && kHwCheck + 1 == KVM_HANDLE_WORDS, "handle layout");
constexpr int64_t kHandleMagic = 0x4b564d4f56453034LL;  // "KVMOVE04"
constexpr int64_t kHandleHasIpc = 1;                    // flag: words 8..15 hold an exported IPC handle
// The flags word carries the flags in its low byte and, above it, the runtime's id of the
// allocation in the exporting process (HIP_POINTER_ATTRIBUTE_BUFFER_ID: every allocation of
// a process gets a new one).  Together with (pid, base, size) it says whether two handles
// name the same allocation; the bytes of hipIpcMemHandle_t do not -- two exports of one
// allocation differ in bytes the runtime leaves unset.
constexpr int kHandleSerialShift = 8;

int64_t handle_check(const int64_t *h)
{
    uint64_t x = 0x5a5a5a5a5a5a5a5aull;
    for (int i = 0; i < kHwCheck; ++i) x = ((x << 7) | (x >> 57)) ^ (uint64_t)h[i];
    return (int64_t)x;
}

// A random word drawn once per process.  A handle is "this process's own", and resolves to
// its pointer without any mapping, only when pid AND nonce match: two processes in different
// pid namespaces (two containers that are both pid 1) share a pid but not a nonce.
int64_t process_nonce()
{
    static const int64_t nonce = [] {
        uint64_t x = 0;
        if (FILE *f = fopen("/dev/urandom", "rb")) {
            if (fread(&x, sizeof x, 1, f) != 1) x = 0;
            fclose(f);
        }
        timespec ts{};
        clock_gettime(CLOCK_MONOTONIC, &ts);
        x ^= ((uint64_t)getpid() << 32) ^ (uint64_t)ts.tv_nsec ^ ((uint64_t)ts.tv_sec << 20) ^ (uint64_t)(uintptr_t)&x;
        return (int64_t)(x | 1);
    }();
    return nonce;
}

bool is_own_handle(const int64_t *h) { return h[kHwPid] == (int64_t)getpid() && h[kHwNonce] == process_nonce(); }

// ---- kernel table

using KernelFn = void (*)(const MigrateArgs);

struct Variant {
    int threads, unroll, flags;
    KernelFn fn[2];         // any shape; [1] reads the packed index table
    KernelFn simple_fn[2];  // one collapsed segment of full tiles
};

#define KVM_VARIANT(T, U, F)                                                                     \
    {T, U, F, {kvm_copy_kernel<u32x4, T, U, F, false>, kvm_copy_kernel<u32x4, T, U, F, true>},      \
     {kvm_copy_simple_kernel<u32x4, T, U, F, false>, kvm_copy_simple_kernel<u32x4, T, U, F, true>}}
#define KVM_VARIANT_ROW(T, F) \
    KVM_VARIANT(T, 1, F), KVM_VARIANT(T, 2, F), KVM_VARIANT(T, 4, F), KVM_VARIANT(T, 8, F), KVM_VARIANT(T, 16, F)

// 16-byte-vector flavours that are compiled in: the one the sweeps chose (64 lanes, one
// vector per lane: a single-wave workgroup that moves 1 KiB), and in the exploration build
// the grid the sweeps ran over.
const Variant kVariants[] = {
    KVM_VARIANT(64, 1, 3),
#ifdef KVM_EXPLORE
    KVM_VARIANT(64, 2, 3),    KVM_VARIANT(64, 4, 3),    KVM_VARIANT(64, 8, 3),   KVM_VARIANT(64, 16, 3),
    KVM_VARIANT_ROW(128, 3),  KVM_VARIANT_ROW(256, 3),  KVM_VARIANT_ROW(512, 3), KVM_VARIANT_ROW(1024, 3),
    KVM_VARIANT_ROW(64, 7),   KVM_VARIANT_ROW(128, 7),  KVM_VARIANT_ROW(256, 7),
    KVM_VARIANT_ROW(512, 7),  KVM_VARIANT_ROW(1024, 7),
    KVM_VARIANT(64, 1, 0),    KVM_VARIANT(64, 1, 1),    KVM_VARIANT(64, 1, 2),
    KVM_VARIANT(256, 4, 0),   KVM_VARIANT(256, 4, 1),   KVM_VARIANT(256, 4, 2),
    KVM_VARIANT(256, 8, 0),   KVM_VARIANT(256, 8, 1),   KVM_VARIANT(256, 8, 2),
    KVM_VARIANT(512, 8, 0),
#endif
};

struct Launch {
    KernelFn fn = nullptr;
    KernelFn simple_fn = nullptr;
    int threads = 0;
    int unroll = 0;
    int vec = 0;
};

int pick_kernel(int vec, bool packed, Launch *l)
{
    l->vec = vec;
    if (vec != 16) {
        // narrow vectors only serve odd shapes and misaligned pools: one flavour each
        l->threads = 256;
        l->unroll = 4;
        l->fn = vec == 8 ? (packed ? kvm_copy_kernel<u32x2, 256, 4, 3, true> : kvm_copy_kernel<u32x2, 256, 4, 3, false>)
              : vec == 4 ? (packed ? kvm_copy_kernel<uint32_t, 256, 4, 3, true> : kvm_copy_kernel<uint32_t, 256, 4, 3, false>)
              : vec == 2 ? (packed ? kvm_copy_kernel<uint16_t, 256, 4, 3, true> : kvm_copy_kernel<uint16_t, 256, 4, 3, false>)
                         : (packed ? kvm_copy_kernel<uint8_t, 256, 4, 3, true> : kvm_copy_kernel<uint8_t, 256, 4, 3, false>);
        return KVM_OK;
    }
#ifdef KVM_EXPLORE
    const int threads = (int)opt_threads.load(), unroll = (int)opt_unroll.load();
    const int flags = (opt_nt_load.load() ? kNtLoad : 0) | (opt_nt_store.load() ? kNtStore : 0) |
                      (opt_wave_contig.load() ? kWaveContig : 0);
#else
    const int threads = 64, unroll = 1, flags = kNtLoad | kNtStore;
#endif
    for (const Variant &v : kVariants) {
        if (v.threads == threads && v.unroll == unroll && v.flags == flags) {
            l->threads = threads;
            l->unroll = unroll;
            l->fn = v.fn[packed];
            l->simple_fn = v.simple_fn[packed];
            return KVM_OK;
        }
    }
    return fail(KVM_EINVAL, "no kernel was built for threads=%d unroll=%d nt_load=%d nt_store=%d wave_contig=%d",
                threads, unroll, flags & 1, (flags >> 1) & 1, (flags >> 2) & 1);
}

int vec_width(uint64_t bits)
{
    // largest power of two <= 16 dividing every address and stride OR-ed into `bits`
    for (int v = 16; v > 1; v >>= 1)
        if ((bits & (uint64_t)(v - 1)) == 0) return v;
    return 1;
}

// Multiplier and shifts with which fast_div divides by d (d >= 1).
void make_magic(uint32_t d, uint32_t *magic, uint32_t *shifts)
{
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;                      // 2^(l-1) < d <= 2^l
    const uint64_t m = ((1ull << 32) * ((1ull << l) - d)) / d + 1;
    const uint32_t sh1 = l < 1 ? l : 1, sh2 = l - sh1;
    *magic = (uint32_t)m;
    *shifts = sh1 | (sh2 << 8);
}

// Splits a segment's rows into workgroup tiles of about tile_bytes.
void tile_segment(Seg &s, uint32_t tile_bytes, uint32_t *tiles)
{
    if (s.run_bytes >= tile_bytes) {
        s.rows_per_tile = 1;
        s.piece_bytes = tile_bytes;
        s.pieces_per_row = (s.run_bytes + tile_bytes - 1) / tile_bytes;
        *tiles = s.n_rows * s.pieces_per_row;
    } else {
        s.rows_per_tile = std::max<uint32_t>(1, tile_bytes / s.run_bytes);
        s.rows_per_tile = std::min(s.rows_per_tile, s.n_rows);
        s.piece_bytes = s.run_bytes;
        s.pieces_per_row = 1;
        *tiles = (s.n_rows + s.rows_per_tile - 1) / s.rows_per_tile;
    }
    make_magic(s.pieces_per_row, &s.pieces_magic, &s.pieces_shifts);
}

// Folds rows that are back to back on both sides into one long run.
void collapse(Seg &s)
{
    if (s.n_rows > 1 && s.run_bytes == s.src_row_stride && s.run_bytes == s.dst_row_stride &&
        (uint64_t)s.run_bytes * s.n_rows < (1ull << 32)) {
        s.run_bytes *= s.n_rows;
        s.src_row_stride = s.dst_row_stride = s.run_bytes;
        s.n_rows = 1;
    }
}

struct Plan {
    std::vector<Seg> segs;         // untiled
    int64_t min_src_blocks = 0;    // smallest block count over the pools that are read
    uint64_t dst_block_stride = 0;
    int vec = 16;
    int64_t payload_per_block = 0; // K+V bytes this rank receives per block
};

int check_geom(const KvmGeom *g)
{
    if (!g) return fail(KVM_EINVAL, "geometry is null");
    if (g->num_layers <= 0 || g->num_kv_heads <= 0 || g->block_size <= 0 || g->head_dim <= 0 ||
        g->dtype_bytes <= 0)
        return fail(KVM_EINVAL, "geometry has a non-positive dimension");
    if (g->ctx_pp_size <= 0 || g->ctx_tp_size <= 0 || g->dec_pp_size <= 0 || g->dec_tp_size <= 0)
        return fail(KVM_EINVAL, "parallel sizes must be positive");
    if (g->dec_pp_rank < 0 || g->dec_pp_rank >= g->dec_pp_size || g->dec_tp_rank < 0 ||
        g->dec_tp_rank >= g->dec_tp_size)
        return fail(KVM_EINVAL, "decoding rank (pp %d, tp %d) outside (pp %d, tp %d)", g->dec_pp_rank,
                    g->dec_tp_rank, g->dec_pp_size, g->dec_tp_size);
    // distserve/config.py:281-285 and :252-256 assert the same divisibility
    if (g->num_layers % g->ctx_pp_size || g->num_layers % g->dec_pp_size)
        return fail(KVM_EINVAL, "num_layers %lld not divisible by a pipeline size (%d, %d)",
                    (long long)g->num_layers, g->ctx_pp_size, g->dec_pp_size);
    if (g->num_kv_heads % g->ctx_tp_size || g->num_kv_heads % g->dec_tp_size)
        return fail(KVM_EINVAL, "num_kv_heads %lld not divisible by a tensor size (%d, %d)",
                    (long long)g->num_kv_heads, g->ctx_tp_size, g->dec_tp_size);
    return KVM_OK;
}

// `arithmetic_only`: context ranks that are not registered count as 16-byte aligned pools of
// unknown size at address 0, so that the launch shape can be computed without a device.
// The caller holds g_mu (shared) and keeps it until the plan's pointers are no longer used.
int build_plan(const KvmGeom *g, const void *dst_k, const void *dst_v, Plan *plan, bool arithmetic_only = false)
{
    if (int rc = check_geom(g)) return rc;
    const int64_t Lc = g->num_layers / g->ctx_pp_size, Hc = g->num_kv_heads / g->ctx_tp_size;
    const int64_t Ld = g->num_layers / g->dec_pp_size, Hd = g->num_kv_heads / g->dec_tp_size;
    const int64_t head_bytes = g->block_size * g->head_dim * g->dtype_bytes;
    const int64_t l0 = g->dec_pp_rank * Ld, l1 = l0 + Ld;
    const int64_t h0 = g->dec_tp_rank * Hd, h1 = h0 + Hd;
    const int64_t src_block = Lc * Hc * head_bytes, dst_block = Ld * Hd * head_bytes;
    if (src_block >= (1ll << 32) || dst_block >= (1ll << 32))
        return fail(KVM_EINVAL, "a block of %lld bytes is beyond the 4 GiB this kernel addresses",
                    (long long)std::max(src_block, dst_block));

    plan->segs.clear();
    plan->dst_block_stride = (uint64_t)dst_block;
    plan->payload_per_block = 2 * dst_block;
    plan->min_src_blocks = INT64_MAX;
    uint64_t align_bits = (uint64_t)head_bytes | (uint64_t)(uintptr_t)dst_k | (uint64_t)(uintptr_t)dst_v;

    for (int64_t p = l0 / Lc; p * Lc < l1; ++p) {
        for (int64_t t = h0 / Hc; t * Hc < h1; ++t) {
            auto it = g_sources.find(SourceKey{g->ctx_instance, (int32_t)p, (int32_t)t});
            if (it == g_sources.end() && !arithmetic_only)
                return fail(KVM_ENOTREG, "context rank (pp %lld, tp %lld) of context instance %lld is not registered",
                            (long long)p, (long long)t, (long long)g->ctx_instance);
            const Source unknown{g->ctx_pp_size, g->ctx_tp_size, g->num_layers, g->num_kv_heads, nullptr, nullptr,
                                 (int64_t)INT32_MAX * src_block, nullptr, nullptr};
            const Source &src = it == g_sources.end() ? unknown : it->second;
            if (src.ctx_pp_size != g->ctx_pp_size || src.ctx_tp_size != g->ctx_tp_size ||
                src.num_layers != g->num_layers || src.num_kv_heads != g->num_kv_heads)
                return fail(KVM_EMISMATCH,
                            "context rank (pp %lld, tp %lld) was registered for pp %d tp %d L %lld H %lld, "
                            "call says pp %d tp %d L %lld H %lld",
                            (long long)p, (long long)t, src.ctx_pp_size, src.ctx_tp_size,
                            (long long)src.num_layers, (long long)src.num_kv_heads, g->ctx_pp_size,
                            g->ctx_tp_size, (long long)g->num_layers, (long long)g->num_kv_heads);
            if (src.nbytes % src_block)
                return fail(KVM_EMISMATCH,
                            "context pool (pp %lld, tp %lld) of %lld bytes is not a whole number of %lld-byte blocks",
                            (long long)p, (long long)t, (long long)src.nbytes, (long long)src_block);
            plan->min_src_blocks = std::min(plan->min_src_blocks, src.nbytes / src_block);

            const int64_t la = std::max(l0, p * Lc), lb = std::min(l1, (p + 1) * Lc);
            const int64_t ha = std::max(h0, t * Hc), hb = std::min(h1, (t + 1) * Hc);
            const int64_t src_off = ((la - p * Lc) * Hc + (ha - t * Hc)) * head_bytes;
            Seg s{};
            s.src_k = src.k + src_off;
            s.src_v = src.v + src_off;
            s.src_block_stride = (uint64_t)src_block;
            s.src_row_stride = (uint32_t)(Hc * head_bytes);
            s.dst_row_stride = (uint32_t)(Hd * head_bytes);
            s.dst_off = (uint32_t)(((la - l0) * Hd + (ha - h0)) * head_bytes);
            s.run_bytes = (uint32_t)((hb - ha) * head_bytes);
            s.n_rows = (uint32_t)(lb - la);
            collapse(s);
            plan->segs.push_back(s);
            align_bits |= (uint64_t)(uintptr_t)src.k | (uint64_t)(uintptr_t)src.v;
        }
    }
    plan->vec = vec_width(align_bits);
    return KVM_OK;
}

// Fills the second header record: the id -> work item mapping for `tiles` tiles per block.
void plan_work(MigrateArgs &args, uint32_t tiles, uint32_t tile_bytes, bool neighbours)
{
    const uint32_t work = tiles * args.nidx;
    args.tiles_per_block = tiles;
    make_magic(tiles, &args.tiles_magic, &args.tiles_shifts);
    args.work = work;
    int64_t mode = opt_xcd_map.load();
    // Blocks that lie next to each other in the context pool (lists as a block manager hands
    // them out while its free list is still in order) copy 1-5 % faster with the ids in order,
    // scattered blocks 1-2 % faster with every XCD on chunks of its own: measured on all three
    // layouts of the bench, one call per request and one per batch.
    if (mode == 1 && neighbours) mode = 0;
    uint32_t chunk = 0;
    if (mode != 0 && work >= 64) {
        // an eighth of a block per XCD when that is at least 256 KiB, else an eighth of the launch
        const bool block_eighth = tiles % 8 == 0 && (mode == 3 || (mode == 1 && (uint64_t)(tiles / 8) * tile_bytes >= (256u << 10)));
        chunk = block_eighth ? tiles / 8 : (work + 7) / 8;
    }
    args.chunk_tiles = chunk;
    if (chunk == 0) {
        args.chunk_magic = args.chunk_shifts = 0;
        args.work_padded = work;
    } else {
        make_magic(chunk, &args.chunk_magic, &args.chunk_shifts);
        args.work_padded = (work + 8 * chunk - 1) / (8 * chunk) * (8 * chunk);
    }
}

using WalkFn = void (*)(const MigrateArgs, uint32_t);

// The link-bound form's workgroup: 256 lanes that move one 16-byte vector each per step
// (4 KiB per workgroup in flight; narrower vectors move four per lane to keep about as many
// bytes in flight).  Many light workgroups fill the link as well as few heavy ones with the
// same bytes in flight, and disturb HBM-bound kernels beside them less: measured at the
// LLaMA-2-7B slab size, 16 workgroups of 4 KiB against 8 to 10 of 16 KiB: the same 99 % of the
// link alone, a migration beside a swap-in 2.4 % slower instead of 8.6 %, and 46 GB/s each
// way instead of 34 / 49 when a swap-out and a swap-in are in flight together.
WalkFn pick_walk(int vec, bool packed, int *threads, int *unroll)
{
    *threads = 256;
    *unroll = vec == 16 ? 1 : 4;
#ifdef KVM_EXPLORE
    // other workgroup shapes, 16-byte vectors and packed tables only
    if (vec == 16 && packed) {
        const int64_t t = opt_swap_threads.load(), u = opt_swap_unroll.load();
        WalkFn fn = nullptr;
#define KVM_WALK(T, U) if (t == T && u == U) fn = kvm_walk_kernel<u32x4, true, T, U>;
        KVM_WALK(64, 1) KVM_WALK(64, 2) KVM_WALK(64, 4) KVM_WALK(128, 1) KVM_WALK(128, 2) KVM_WALK(128, 4)
        KVM_WALK(256, 2) KVM_WALK(256, 4) KVM_WALK(256, 8) KVM_WALK(512, 4) KVM_WALK(1024, 4)
#undef KVM_WALK
        if (fn) {
            *threads = (int)t;
            *unroll = (int)u;
            return fn;
        }
    }
#endif
    if (packed)
        return vec == 16 ? kvm_walk_kernel<u32x4, true, 256, 1>
             : vec == 8  ? kvm_walk_kernel<u32x2, true, 256, 4>
             : vec == 4  ? kvm_walk_kernel<uint32_t, true, 256, 4>
             : vec == 2  ? kvm_walk_kernel<uint16_t, true, 256, 4>
                         : kvm_walk_kernel<uint8_t, true, 256, 4>;
    return vec == 16 ? kvm_walk_kernel<u32x4, false, 256, 1>
         : vec == 8  ? kvm_walk_kernel<u32x2, false, 256, 4>
         : vec == 4  ? kvm_walk_kernel<uint32_t, false, 256, 4>
         : vec == 2  ? kvm_walk_kernel<uint16_t, false, 256, 4>
                     : kvm_walk_kernel<uint8_t, false, 256, 4>;
}

// Everything launch_copy decides about one group of up to 8 segments before it launches.
struct Group {
    MigrateArgs args;        // filled up to the index pairs
    uint32_t tiles = 0;      // tiles per block of one pool kind
    int64_t per_launch = 0;  // index pairs per launch
    bool simple = false;
};

// A launch is a 1-D grid of 2 * work_padded workgroups of `threads` lanes, and the runtime
// refuses a grid of 2^32 work-items or more.  plan_work pads the work of a launch by fewer
// than 8 tiles, or not at all, so this many index pairs per launch stay below that.
int64_t pairs_per_launch(uint32_t tiles, int threads, bool packed)
{
    const int64_t max_tiles = (int64_t)(UINT32_MAX / (2u * (uint32_t)threads)) - 8;
    const int64_t table = std::min<int64_t>(packed ? kMaxIdxPacked : kMaxIdx, tune_max_pairs());
    return std::min<int64_t>(table, max_tiles / (int64_t)tiles);
}

// What launch_copy reports about the launches of a call.
struct CopyShape {
    int64_t launches = 0;
    int64_t wgs_per_block = 0;     // workgroups per block, K and V together
    int64_t max_items = 0;         // work-items of the largest launch
    int64_t pairs_per_launch = 0;  // index pairs the largest launch carries at most
    int threads = 0, unroll = 0;
    bool simple = false;           // the short-prologue kernel serves every launch
};

// Enqueues the copy over `segs` x `pairs`, as many launches as the 4 KiB argument needs
// (8 segments and 864 packed or 432 wide index pairs each) and the grid limit allows.  Every
// launch of the call is sized and checked before the first one is enqueued, so a call that
// cannot be launched has touched nothing.  `pairs == nullptr` only counts what would be
// launched.  `packed`: every index is below 65536.  walk_wgs > 0 selects the link-bound form
// with that many workgroups per pool kind.
int launch_copy(std::vector<Seg> segs, const IdxPair *pairs, int64_t n, bool packed, char *dst_k, char *dst_v,
                uint64_t dst_block_stride, int vec, hipStream_t stream, CopyShape *shape = nullptr,
                int walk_wgs = 0, bool neighbours = false)
{
    packed = packed && tune_packed();
    Launch k;
    if (int rc = pick_kernel(vec, packed, &k)) return rc;
    // tile_bytes 0 = one shot: exactly what the workgroup's lanes hold in flight
    uint32_t tile_bytes = (uint32_t)tune_tile_bytes();
    WalkFn walk_fn = nullptr;
    int walk_threads = 256, walk_unroll = 4;
    if (walk_wgs > 0) walk_fn = pick_walk(vec, packed, &walk_threads, &walk_unroll);
    if (tile_bytes == 0) tile_bytes = (uint32_t)((walk_wgs > 0 ? walk_threads * walk_unroll : k.threads * k.unroll) * vec);
    CopyShape out;
    out.threads = k.threads;
    out.unroll = k.unroll;
    out.simple = !segs.empty();
    std::vector<Group> groups((segs.size() + kMaxSegs - 1) / kMaxSegs);
    for (size_t gi = 0; gi < groups.size(); ++gi) {
        const size_t s0 = gi * kMaxSegs;
        Group &grp = groups[gi];
        MigrateArgs &args = grp.args;
        args.dst_k = dst_k;
        args.dst_v = dst_v;
        args.dst_block_stride = dst_block_stride;
        args.nseg = (uint32_t)std::min<size_t>(kMaxSegs, segs.size() - s0);
        uint64_t tiles_total = 0;
        for (uint32_t j = 0; j < args.nseg; ++j) {
            Seg s = segs[s0 + j];
            uint32_t tiles = 0;
            tile_segment(s, tile_bytes, &tiles);
            tiles_total += tiles;
            args.tile_end[j] = (uint32_t)std::min<uint64_t>(tiles_total, UINT32_MAX);
            args.seg[j] = s;
        }
        for (uint32_t j = args.nseg; j < kMaxSegs; ++j) args.tile_end[j] = UINT32_MAX;
        args.tile_end[args.nseg - 1] = UINT32_MAX;   // nothing lies past the last segment
        // one collapsed segment of full one-shot tiles takes the short-prologue kernel
        const Seg &first = args.seg[0];
        grp.simple = walk_wgs == 0 && k.simple_fn && tune_simple() && args.nseg == 1 &&
                     first.n_rows == 1 && first.rows_per_tile == 1 && first.run_bytes % tile_bytes == 0 &&
                     tile_bytes == (uint32_t)(k.threads * k.unroll * vec);
        out.simple = out.simple && grp.simple;
        out.wgs_per_block += 2 * (int64_t)tiles_total;
        if (tiles_total == 0 || tiles_total > (1u << 29))
            return fail(KVM_EINVAL, "%llu tiles per block cannot be launched", (unsigned long long)tiles_total);
        grp.tiles = (uint32_t)tiles_total;
        // the walking form's grid is a few workgroups whatever the work
        grp.per_launch = walk_wgs > 0
                             ? std::min<int64_t>(packed ? kMaxIdxPacked : kMaxIdx, (int64_t)(UINT32_MAX / grp.tiles))
                             : pairs_per_launch(grp.tiles, k.threads, packed);
        if (grp.per_launch < 1)
            return fail(KVM_EINVAL, "one block is %u tiles of %d lanes per pool kind: no launch can hold it",
                        grp.tiles, k.threads);
        out.pairs_per_launch = std::max(out.pairs_per_launch, grp.per_launch);
        const int64_t largest = std::min<int64_t>(grp.per_launch, std::max<int64_t>(n, 1));
        if (walk_wgs > 0) {
            out.max_items = std::max<int64_t>(out.max_items, 2 * walk_threads * (int64_t)walk_wgs);
        } else {
            args.nidx = (uint32_t)largest;      // the launch loop below sets it again, launch by launch
            plan_work(args, grp.tiles, tile_bytes, neighbours);
            const int64_t items = 2 * (int64_t)args.work_padded * k.threads;
            if (items > (int64_t)UINT32_MAX)
                return fail(KVM_EINVAL, "a launch of %lld work-items cannot be made", (long long)items);
            out.max_items = std::max(out.max_items, items);
        }
        out.launches += n == 0 ? 1 : (n + grp.per_launch - 1) / grp.per_launch;
    }
    if (pairs) {
        for (Group &grp : groups) {
            MigrateArgs &args = grp.args;
            for (int64_t i0 = 0; i0 < n; i0 += grp.per_launch) {
                args.nidx = (uint32_t)std::min<int64_t>(grp.per_launch, n - i0);
                if (packed) {
                    for (uint32_t i = 0; i < args.nidx; ++i)
                        args.packed[i] = (uint32_t)pairs[i0 + i].ctx | ((uint32_t)pairs[i0 + i].dec << 16);
                } else {
                    memcpy(args.idx, pairs + i0, args.nidx * sizeof(IdxPair));
                }
                if (walk_wgs > 0) {
                    const uint32_t work = grp.tiles * args.nidx;
                    hipLaunchKernelGGL(walk_fn, dim3(std::min<uint32_t>((uint32_t)walk_wgs, work), 2),
                                       dim3(walk_threads), 0, stream, args, grp.tiles);
                } else {
                    plan_work(args, grp.tiles, tile_bytes, neighbours);
                    hipLaunchKernelGGL(grp.simple ? k.simple_fn : k.fn, dim3(2 * args.work_padded), dim3(k.threads),
                                       (size_t)tune_lds_pad(), stream, args);
                }
                KVM_HIP(hipGetLastError());
            }
        }
    }
    if (shape) *shape = out;
    return KVM_OK;
}

// dec index list must not repeat: the copies of one call run concurrently.
thread_local std::vector<uint64_t> g_seen;

// Orders the pairs of a call by source block; pairs with the same source keep their order.
// The copy does not depend on the order of its pairs, the memory system does: a call that
// names a large part of the source pool reads it front to back instead of at random.
thread_local std::vector<uint32_t> g_count;
thread_local std::vector<IdxPair> g_sorted;

void sort_by_source(std::vector<IdxPair> *pairs, int64_t n_src)
{
    const size_t n = pairs->size();
    if ((uint64_t)n_src > 8 * (uint64_t)n + 1024) {
        std::stable_sort(pairs->begin(), pairs->end(), [](const IdxPair &x, const IdxPair &y) { return x.ctx < y.ctx; });
        return;
    }
    // counting sort: O(n + n_src)
    g_count.assign((size_t)n_src + 1, 0);
    for (const IdxPair &p : *pairs) ++g_count[(size_t)p.ctx + 1];
    for (size_t b = 0; b < (size_t)n_src; ++b) g_count[b + 1] += g_count[b];
    g_sorted.resize(n);
    for (const IdxPair &p : *pairs) g_sorted[g_count[(size_t)p.ctx]++] = p;
    pairs->swap(g_sorted);
}

// Validates the two lists and turns them into pairs.  `sort` (migration only): the pairs may
// be handed to the kernel in another order than the caller's (option "sort_pairs").
// `neighbours` (optional): whether at least half of the source blocks, in the order the
// kernel gets them, follow their predecessor directly, i.e. the list is mostly runs of
// adjacent blocks.
int check_indices(const int64_t *src, const int64_t *dst, int64_t n, int64_t n_src, int64_t n_dst,
                  const char *src_name, const char *dst_name, std::vector<IdxPair> *pairs,
                  bool sort = false, bool *neighbours = nullptr)
{
    if (n_dst > INT32_MAX || n_src > INT32_MAX)
        return fail(KVM_EINVAL, "pools of more than 2^31 blocks are not supported");
    g_seen.assign((size_t)((n_dst + 63) / 64), 0);
    pairs->resize((size_t)n);
    int64_t adjacent = 0;
    bool ascending = true;
    for (int64_t i = 0; i < n; ++i) {
        const int64_t a = src[i], b = dst[i];
        if (a < 0 || a >= n_src)
            return fail(KVM_ERANGE, "%s[%lld] = %lld is outside [0, %lld)", src_name, (long long)i,
                        (long long)a, (long long)n_src);
        if (b < 0 || b >= n_dst)
            return fail(KVM_ERANGE, "%s[%lld] = %lld is outside [0, %lld)", dst_name, (long long)i,
                        (long long)b, (long long)n_dst);
        uint64_t &w = g_seen[(size_t)(b >> 6)];
        const uint64_t bit = 1ull << (b & 63);
        if (w & bit)
            return fail(KVM_EDUP, "%s names block %lld twice", dst_name, (long long)b);
        w |= bit;
        (*pairs)[(size_t)i] = IdxPair{(int32_t)a, (int32_t)b};
        if (i > 0 && a == src[i - 1] + 1) ++adjacent;
        if (i > 0 && a < src[i - 1]) ascending = false;
    }
    // Sorting pays when the call names a large part of the source pool (measured: +4 % on
    // calls of 800 of 1024 blocks whose rows are half read, +1 % on 1168 of 2048, nothing on
    // 136 of 1024), and costs host time otherwise: a quarter of the pool is the line.
    const int64_t mode = sort ? opt_sort_pairs.load() : 0;
    if (!ascending && (mode == 2 || (mode == 1 && n >= 64 && 4 * n >= n_src))) {
        sort_by_source(pairs, n_src);
        adjacent = 0;
        for (int64_t i = 1; i < n; ++i) adjacent += (*pairs)[(size_t)i].ctx == (*pairs)[(size_t)i - 1].ctx + 1;
    }
    if (neighbours) *neighbours = n > 1 && 2 * adjacent >= n - 1;
    return KVM_OK;
}

int device_of(const void *p, const char *what, int *device)
{
    hipPointerAttribute_t at;
    hipError_t e = hipPointerGetAttributes(&at, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(KVM_EINVAL, "%s (%p) is not memory HIP knows: %s", what, p, hipGetErrorString(e));
    }
    if (at.type != hipMemoryTypeDevice)
        return fail(KVM_EINVAL, "%s (%p) is not device memory", what, p);
    *device = at.device;
    return KVM_OK;
}

int host_pinned(const void *p, const char *what)
{
    hipPointerAttribute_t at;
    hipError_t e = hipPointerGetAttributes(&at, p);
    if (e != hipSuccess || at.type != hipMemoryTypeHost) {
        (void)hipGetLastError();
        return fail(KVM_EINVAL, "%s (%p) is not pinned host memory", what, p);
    }
    return KVM_OK;
}

// Bytes from p to the end of the allocation that holds it, 0 when the runtime cannot tell
// (memory it did not allocate as one range).  A pool that claims more than this would send
// a kernel past mapped memory, so callers refuse it on the host.
uint64_t extent_of(const void *p)
{
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)p) != hipSuccess || !base) {
        (void)hipGetLastError();
        return 0;
    }
    const char *end = (const char *)base + size;
    return end > (const char *)p ? (uint64_t)(end - (const char *)p) : 0;
}

int check_extent(const void *p, uint64_t need, uint64_t extent, const char *what)
{
    if (extent != 0 && need > extent)
        return fail(KVM_ERANGE, "%s (%p) is said to hold %llu bytes but its allocation ends after %llu", what, p,
                    (unsigned long long)need, (unsigned long long)extent);
    return KVM_OK;
}

// A pool argument is looked up afresh on every call: the two runtime queries cost well under a
// microsecond each, and an address remembered from an earlier call may by now belong to another,
// smaller allocation.
int checked_pool(const void *p, uint64_t need, bool on_device, const char *what)
{
    int dev = -1;
    if (on_device) {
        if (int rc = device_of(p, what, &dev)) return rc;
    } else {
        if (int rc = host_pinned(p, what)) return rc;
    }
    return check_extent(p, need, extent_of(p), what);
}

// A second stream (default priority) and the two events that fork it from and join it back
// into the caller's stream; one set per device and direction (so that a swap-out and a
// swap-in issued on different streams still overlap), made on first use, kept until the
// process ends.
struct Fork {
    hipStream_t side = nullptr;
    hipEvent_t forked = nullptr, joined = nullptr;
    std::mutex in_use;   // held while one call forks, enqueues and joins: the events are per set
};
std::mutex g_fork_mu;    // guards the map only (std::map keeps its nodes where they are)
std::map<std::pair<int, bool>, Fork> g_forks;

int get_fork(bool is_swap_in, Fork **out)
{
    int dev = 0;
    KVM_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_fork_mu);
    Fork &f = g_forks[{dev, is_swap_in}];
    if (!f.side) {
        KVM_HIP(hipStreamCreateWithFlags(&f.side, hipStreamNonBlocking));
        KVM_HIP(hipEventCreateWithFlags(&f.forked, hipEventDisableTiming));
        KVM_HIP(hipEventCreateWithFlags(&f.joined, hipEventDisableTiming));
    }
    *out = &f;
    return KVM_OK;
}

// Which implementation serves a swap call (0, 1 or 2; see the "swap_mode" option).  Mode 3
// takes the copy kernel unless the call's copies average "swap_kernel_below" bytes or more: the
// kernel fills 97-100 % of the link at every slab size for a tenth of a millisecond of host
// time per call, where the copy engines need 2 MiB and more per copy to hide their per-copy
// cost (4 MiB copies 98 % of the link, 1 MiB 85-91 %, 288 KiB 55 %, 64 KiB 20 %) and two
// runtime calls per block (4-5 ms for 2048 blocks).  *out_runs = copies per pool.
int64_t swap_mode_for(const IdxPair *pairs, int64_t n, int64_t slab_bytes, int64_t *out_runs)
{
    int64_t runs = n > 0 ? 1 : 0;
    for (int64_t i = 1; i < n; ++i)
        runs += !(pairs[i].ctx == pairs[i - 1].ctx + 1 && pairs[i].dec == pairs[i - 1].dec + 1);
    if (out_runs) *out_runs = runs;
    const int64_t mode = opt_swap_mode.load();
    if (mode != 3) return mode;
    return runs > 0 && (n * slab_bytes) / runs < opt_swap_kernel_below.load() ? 1 : 2;
}

// ---- memory handles and bindings

// What a handle resolves to in this process.
struct Resolved {
    const char *ptr = nullptr;
    int64_t nbytes = 0;
    const char *map = nullptr;   // local base of the other process's allocation, null for a pool of this process
};

// Unmaps the mappings `doomed` selects, after dropping the pools bound through them and after
// the device has finished whatever may still read them.  The caller holds g_reg_mu.
template <typename Pred>
int close_mappings(Pred doomed)
{
    bool any = false;
    for (const Opened &o : g_opened) any = any || doomed(o);
    if (!any) return KVM_OK;
    int rc = KVM_OK;
    std::unique_lock<std::shared_mutex> lock(g_mu);   // no migrate call is between its lookup and its launch
    for (const Opened &o : g_opened) {
        if (!doomed(o)) continue;
        for (auto it = g_sources.begin(); it != g_sources.end();)
            it = (it->second.map_k == o.local_base || it->second.map_v == o.local_base) ? g_sources.erase(it) : ++it;
    }
    if (hipDeviceSynchronize() != hipSuccess) {
        (void)hipGetLastError();
        rc = fail(KVM_EHIP, "the device did not become idle before a mapping was closed");
    }
    for (size_t i = 0; i < g_opened.size();) {
        if (!doomed(g_opened[i])) {
            ++i;
            continue;
        }
        const hipError_t e = hipIpcCloseMemHandle(g_opened[i].local_base);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            rc = fail(KVM_EHIP, "hipIpcCloseMemHandle failed: %s", hipGetErrorString(e));
        }
        g_opened.erase(g_opened.begin() + (ptrdiff_t)i);
    }
    return rc;
}

// Mappings that no registered pool lies in any more (a binding was replaced, a registration
// failed half way): they would keep the exporter's freed memory pinned.
int close_unreferenced_mappings()
{
    std::vector<const char *> used;
    {
        std::shared_lock<std::shared_mutex> lock(g_mu);
        for (const auto &kv : g_sources) {
            if (kv.second.map_k) used.push_back(kv.second.map_k);
            if (kv.second.map_v) used.push_back(kv.second.map_v);
        }
    }
    return close_mappings([&used](const Opened &o) {
        return std::find(used.begin(), used.end(), (const char *)o.local_base) == used.end();
    });
}

// Resolves a handle to a pointer valid in this process, mapping the exporter's allocation
// if it is another process's and not mapped yet.  The caller holds g_reg_mu.
int open_handle(const int64_t *h, const char *what, Resolved *out)
{
    if (!h) return fail(KVM_EINVAL, "%s handle is null", what);
    if (h[kHwMagic] != kHandleMagic || h[kHwCheck] != handle_check(h))
        return fail(KVM_EHANDLE, "%s handle is not a kvmove memory handle", what);
    if (h[kHwBytes] <= 0 || h[kHwPtr] == 0)
        return fail(KVM_EHANDLE, "%s handle names no memory", what);
    out->nbytes = h[kHwBytes];
    out->map = nullptr;
    if (is_own_handle(h)) {
        out->ptr = (const char *)(uintptr_t)h[kHwPtr];
        return KVM_OK;
    }
    if (!(h[kHwFlags] & kHandleHasIpc)) {
        if (h[kHwAllocSize] >= KVM_IPC_MAX_ALLOC_BYTES)
            return fail(KVM_EHANDLE,
                        "%s handle of process %lld names a pool inside an allocation of %lld bytes; allocations of "
                        "%lld bytes and more are not shared between processes",
                        what, (long long)h[kHwPid], (long long)h[kHwAllocSize], (long long)KVM_IPC_MAX_ALLOC_BYTES);
        return fail(KVM_EHANDLE, "%s handle of process %lld was not exported for other processes", what,
                    (long long)h[kHwPid]);
    }
    const int64_t off = h[kHwPtr] - h[kHwAllocBase];
    if (h[kHwAllocSize] <= 0 || h[kHwAllocSize] >= KVM_IPC_MAX_ALLOC_BYTES || off < 0 ||
        off + h[kHwBytes] > h[kHwAllocSize])
        return fail(KVM_EHANDLE, "%s handle of process %lld is inconsistent (pool at offset %lld, %lld bytes, in an "
                    "allocation of %lld)", what, (long long)h[kHwPid], (long long)off, (long long)h[kHwBytes],
                    (long long)h[kHwAllocSize]);
    hipIpcMemHandle_t ipc;
    memcpy(&ipc, &h[kHwIpc], sizeof ipc);
    const int64_t serial = (int64_t)((uint64_t)h[kHwFlags] >> kHandleSerialShift);
    for (const Opened &o : g_opened) {
        if (o.pid != h[kHwPid] || o.nonce != h[kHwNonce] || o.remote_base != h[kHwAllocBase]) continue;
        // The same allocation: its id matches, or -- where the exporter had no id to give -- it
        // was mapped by this very registration call (a rank's K and V pools in one allocation).
        // A mapping without an id is never trusted across calls: the exporter may have freed
        // the memory and allocated anew at the same address.
        if (serial != 0 ? o.serial == serial : (o.serial == 0 && o.opened_in == g_reg_call)) {
            if (o.size != h[kHwAllocSize])
                return fail(KVM_EHANDLE, "%s handle of process %lld says its allocation holds %lld bytes, the same "
                            "allocation is open with %lld", what, (long long)h[kHwPid], (long long)h[kHwAllocSize],
                            (long long)o.size);
            out->ptr = o.local_base + off;
            out->map = o.local_base;
            return KVM_OK;
        }
        // The exporting process has made a new allocation at the old address (or may have): the
        // old mapping and every pool bound through it are stale.
        const char *stale = o.local_base;
        if (int rc = close_mappings([stale](const Opened &x) { return x.local_base == stale; })) return rc;
        break;
    }
    void *local = nullptr;
    const hipError_t e = hipIpcOpenMemHandle(&local, ipc, hipIpcMemLazyEnablePeerAccess);
    if (e != hipSuccess || !local) {
        (void)hipGetLastError();
        return fail(KVM_EHANDLE, "%s handle of process %lld could not be opened: %s", what, (long long)h[kHwPid],
                    hipGetErrorString(e));
    }
    // The size in the handle is the exporter's word; where the runtime can tell how much it
    // has mapped, a handle that claims more is refused before a kernel could run off the end.
    const uint64_t mapped = extent_of(local);
    if (mapped != 0 && mapped < (uint64_t)h[kHwAllocSize]) {
        (void)hipIpcCloseMemHandle(local);
        return fail(KVM_EHANDLE, "%s handle of process %lld says its allocation holds %lld bytes, the mapping holds %llu",
                    what, (long long)h[kHwPid], (long long)h[kHwAllocSize], (unsigned long long)mapped);
    }
    g_opened.push_back(Opened{h[kHwPid], h[kHwNonce], h[kHwAllocBase], h[kHwAllocSize], serial, g_reg_call, (char *)local});
    out->ptr = (char *)local + off;
    out->map = (char *)local;
    return KVM_OK;
}

int check_source_args(int32_t ctx_pp_size, int32_t ctx_tp_size, int32_t pp_rank, int32_t tp_rank,
                             int64_t num_layers, int64_t num_kv_heads, const void *k_base, const void *v_base,
                             int64_t nbytes_each)
{
    if (!k_base || !v_base || nbytes_each <= 0)
        return fail(KVM_EINVAL, "kvm_register_source: null pool or non-positive size");
    if (ctx_pp_size <= 0 || ctx_tp_size <= 0 || pp_rank < 0 || pp_rank >= ctx_pp_size || tp_rank < 0 ||
        tp_rank >= ctx_tp_size)
        return fail(KVM_EINVAL, "context rank (pp %d, tp %d) outside (pp %d, tp %d)", pp_rank, tp_rank,
                    ctx_pp_size, ctx_tp_size);
    if (num_layers <= 0 || num_kv_heads <= 0 || num_layers % ctx_pp_size || num_kv_heads % ctx_tp_size)
        return fail(KVM_EINVAL, "L %lld / H %lld do not split over pp %d / tp %d", (long long)num_layers,
                    (long long)num_kv_heads, ctx_pp_size, ctx_tp_size);
    return KVM_OK;
}

// A pool of this process: device memory whose allocation holds the bytes it claims.
int check_local_pool(const void *p, int64_t nbytes, const char *what, int *device)
{
    if (int rc = device_of(p, what, device)) return rc;
    return check_extent(p, (uint64_t)nbytes, extent_of(p), what);
}

// Binds one context rank's pools.  Pools that were resolved through a mapping (map != null)
// are device memory of the size their handle states: open_handle has checked that the pool
// lies inside the mapping, and the runtime's own queries may not know a mapping as an
// allocation; every other pointer is checked here.  The caller holds g_reg_mu.
int bind_source(int32_t ctx_pp_size, int32_t ctx_tp_size, int32_t pp_rank, int32_t tp_rank,
                       int64_t num_layers, int64_t num_kv_heads, const Resolved &k, const Resolved &v,
                       int64_t ctx_instance)
{
    if (k.nbytes != v.nbytes)
        return fail(KVM_EMISMATCH, "K pool (%lld bytes) and V pool (%lld bytes) differ", (long long)k.nbytes,
                    (long long)v.nbytes);
    if (int rc = check_source_args(ctx_pp_size, ctx_tp_size, pp_rank, tp_rank, num_layers, num_kv_heads, k.ptr,
                                   v.ptr, k.nbytes))
        return rc;
    int dk = -1, dv = -1;
    if (!k.map)
        if (int rc = check_local_pool(k.ptr, k.nbytes, "context K pool", &dk)) return rc;
    if (!v.map)
        if (int rc = check_local_pool(v.ptr, v.nbytes, "context V pool", &dv)) return rc;
    if (dk >= 0 && dv >= 0 && dk != dv) return fail(KVM_EINVAL, "context K and V pools sit on different devices");
    const Source s{ctx_pp_size, ctx_tp_size, num_layers, num_kv_heads, k.ptr, v.ptr, k.nbytes, k.map, v.map};
    std::unique_lock<std::shared_mutex> lock(g_mu);
    g_sources[SourceKey{ctx_instance, pp_rank, tp_rank}] = s;
    return KVM_OK;
}

// Whether a call's index pairs fit the packed table: every index is below its pool's block
// count, so pools of at most 65536 blocks make every index fit 16 bits.
bool fits_packed(int64_t n_src, int64_t n_dst) { return n_src <= 65536 && n_dst <= 65536; }

}  // namespace

// ------------------------------------------------------------------------- C ABI

extern "C" {

int kvm_version(void) { return KVM_ABI_MAJOR * 10000 + 0 * 100 + 0; }

const char *kvm_last_error(void) { return g_err.c_str(); }

int kvm_set_option(const char *name, int64_t value)
{
    std::atomic<int64_t> *o = find_opt(name);
    if (!o) return fail(KVM_EINVAL, "unknown option '%s'", name ? name : "(null)");
    bool ok = true;
    if (o == &opt_swap_wgs || o == &opt_swap_wgs_in) ok = value >= 1 && value <= 4096;
    else if (o == &opt_xcd_map) ok = value >= 0 && value <= 3;
    else if (o == &opt_swap_mode) ok = value >= 0 && value <= 3;
    else if (o == &opt_swap_kernel_below) ok = value >= 0 && value <= (1ll << 32);
    else if (o == &opt_sort_pairs) ok = value >= 0 && value <= 2;
#ifdef KVM_EXPLORE
    else if (o == &opt_tile_bytes) ok = value == 0 || (value >= 1024 && value <= (1 << 26) && (value & (value - 1)) == 0);
    else if (o == &opt_threads) ok = value == 64 || value == 128 || value == 256 || value == 512 || value == 1024;
    else if (o == &opt_unroll) ok = value == 1 || value == 2 || value == 4 || value == 8 || value == 16;
    else if (o == &opt_lds_pad) ok = value >= 0 && value <= 65536;
    else if (o == &opt_max_pairs) ok = value >= 1 && value <= kMaxIdxPacked;
    else if (o == &opt_swap_threads) ok = value >= 64 && value <= 1024;
    else if (o == &opt_swap_unroll) ok = value >= 1 && value <= 8;
#endif
    else ok = value == 0 || value == 1;
    if (!ok) return fail(KVM_EINVAL, "value %lld is not valid for option '%s'", (long long)value, name);
    o->store(value);
    return KVM_OK;
}

int64_t kvm_get_option(const char *name)
{
    std::atomic<int64_t> *o = find_opt(name);
    if (!o) return fail(KVM_EINVAL, "unknown option '%s'", name ? name : "(null)");
    return o->load();
}

int kvm_get_mem_handle(const void *dev_ptr, int64_t nbytes, int64_t *out_handle)
{
    if (!dev_ptr || !out_handle || nbytes <= 0)
        return fail(KVM_EINVAL, "kvm_get_mem_handle: null pointer or non-positive size");
    int dev = 0;
    if (int rc = device_of(dev_ptr, "pool", &dev)) return rc;
    int64_t *h = out_handle;
    memset(h, 0, sizeof(int64_t) * KVM_HANDLE_WORDS);
    h[kHwMagic] = kHandleMagic;
    h[kHwPid] = (int64_t)getpid();
    h[kHwDevice] = dev;
    h[kHwPtr] = (int64_t)(uintptr_t)dev_ptr;
    h[kHwBytes] = nbytes;
    h[kHwNonce] = process_nonce();
    // The IPC handle names a whole allocation, so the pool travels as (allocation, offset).
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)dev_ptr) == hipSuccess && base) {
        const uint64_t off = (uint64_t)((const char *)dev_ptr - (const char *)base);
        if (off + (uint64_t)nbytes > (uint64_t)size)
            return fail(KVM_ERANGE, "pool (%p) is said to hold %lld bytes but its allocation ends after %llu",
                        dev_ptr, (long long)nbytes, (unsigned long long)((uint64_t)size - off));
        h[kHwAllocBase] = (int64_t)(uintptr_t)base;
        h[kHwAllocSize] = (int64_t)size;
        if ((int64_t)size < KVM_IPC_MAX_ALLOC_BYTES) {
            hipIpcMemHandle_t ipc;
            memset(&ipc, 0, sizeof ipc);
            if (hipIpcGetMemHandle(&ipc, base) == hipSuccess) {
                memcpy(&h[kHwIpc], &ipc, sizeof ipc);
                h[kHwFlags] |= kHandleHasIpc;
                unsigned long long id = 0;
                if (hipPointerGetAttribute(&id, HIP_POINTER_ATTRIBUTE_BUFFER_ID, base) == hipSuccess)
                    h[kHwFlags] |= (int64_t)((id & 0x7fffffffffffffull) << kHandleSerialShift);
                else
                    (void)hipGetLastError();   // no id: (pid, base, size) alone names the allocation
            } else {
                (void)hipGetLastError();   // stays a handle for this process only
            }
        }
    } else {
        (void)hipGetLastError();
    }
    h[kHwCheck] = handle_check(h);
    return KVM_OK;
}

int kvm_register_source(int32_t ctx_pp_size, int32_t ctx_tp_size, int32_t pp_rank, int32_t tp_rank,
                        int64_t num_layers, int64_t num_kv_heads, const void *k_base,
                        const void *v_base, int64_t nbytes_each, int64_t ctx_instance)
{
    Resolved k, v;
    k.ptr = (const char *)k_base;
    v.ptr = (const char *)v_base;
    k.nbytes = v.nbytes = nbytes_each;
    std::lock_guard<std::mutex> reg(g_reg_mu);
    ++g_reg_call;
    if (int rc = bind_source(ctx_pp_size, ctx_tp_size, pp_rank, tp_rank, num_layers, num_kv_heads, k, v, ctx_instance))
        return rc;
    return close_unreferenced_mappings();   // the binding this one replaced may have been the last in a mapping
}

int kvm_register_mem_handle(const int64_t *k_handle, const int64_t *v_handle, int64_t num_layers,
                            int64_t num_kv_heads, const int64_t context_pc[4],
                            const int64_t decoding_pc[4], int64_t ctx_instance)
{
    if (!context_pc || !decoding_pc) return fail(KVM_EINVAL, "parallel config list is null");
    if (!k_handle || !v_handle) return fail(KVM_EINVAL, "a memory handle is null");
    // [tp_size, tp_rank, pp_size, pp_rank]; the decoding list only has to be well formed here,
    // the decoding rank's rectangle is taken from each migrate call.
    if (decoding_pc[0] <= 0 || decoding_pc[2] <= 0 || decoding_pc[1] < 0 || decoding_pc[1] >= decoding_pc[0] ||
        decoding_pc[3] < 0 || decoding_pc[3] >= decoding_pc[2])
        return fail(KVM_EINVAL, "decoding parallel config [%lld,%lld,%lld,%lld] is malformed",
                    (long long)decoding_pc[0], (long long)decoding_pc[1], (long long)decoding_pc[2],
                    (long long)decoding_pc[3]);
    for (int i = 0; i < 4; ++i)
        if (context_pc[i] < 0 || context_pc[i] > INT32_MAX)
            return fail(KVM_EINVAL, "context parallel config [%lld,%lld,%lld,%lld] is malformed",
                        (long long)context_pc[0], (long long)context_pc[1], (long long)context_pc[2],
                        (long long)context_pc[3]);
    std::lock_guard<std::mutex> reg(g_reg_mu);
    ++g_reg_call;
    Resolved k, v;
    int rc = open_handle(k_handle, "K", &k);
    if (rc == KVM_OK) rc = open_handle(v_handle, "V", &v);
    if (rc == KVM_OK)
        rc = bind_source((int32_t)context_pc[2], (int32_t)context_pc[0], (int32_t)context_pc[3],
                         (int32_t)context_pc[1], num_layers, num_kv_heads, k, v, ctx_instance);
    // Whatever this call mapped and did not bind (the V handle failed after the K handle had
    // opened, the pools disagreed), and whatever the replaced binding leaves unused, goes.
    const std::string text = g_err;
    const int rc_close = close_unreferenced_mappings();
    if (rc != KVM_OK) g_err = text;
    return rc != KVM_OK ? rc : rc_close;
}

int kvm_reset(void)
{
    std::lock_guard<std::mutex> reg(g_reg_mu);
    {
        std::unique_lock<std::shared_mutex> lock(g_mu);
        g_sources.clear();
    }
    // kernels in flight may still read the mappings: close_mappings waits for the device first
    return close_mappings([](const Opened &) { return true; });
}

int64_t kvm_opened_handles(void)
{
    std::lock_guard<std::mutex> reg(g_reg_mu);
    return (int64_t)g_opened.size();
}

int kvm_migrate_plan(const KvmGeom *geom, int64_t n, const void *dst_k, const void *dst_v, int64_t dst_num_blocks,
                     int64_t out[10])
{
    if (!out) return fail(KVM_EINVAL, "out is null");
    if (n < 0) return fail(KVM_EINVAL, "n is negative");
    const bool arithmetic_only = !dst_k && !dst_v;
    Plan plan;
    std::shared_lock<std::shared_mutex> lock(g_mu);
    if (int rc = build_plan(geom, dst_k, dst_v, &plan, arithmetic_only)) return rc;
    // pools that are not registered count as being as large as the destination pool is said to be
    const int64_t n_src = arithmetic_only ? dst_num_blocks : plan.min_src_blocks;
    const bool packed = dst_num_blocks > 0 && fits_packed(n_src, dst_num_blocks);
    CopyShape shape;
    if (int rc = launch_copy(plan.segs, nullptr, n, packed, nullptr, nullptr, plan.dst_block_stride, plan.vec,
                             nullptr, &shape))
        return rc;
    out[0] = shape.wgs_per_block;
    out[1] = shape.threads;
    out[2] = plan.vec;
    out[3] = (int64_t)plan.segs.size();
    out[4] = shape.launches;
    out[5] = plan.payload_per_block;
    out[6] = shape.simple ? 1 : 0;
    out[7] = shape.max_items;
    out[8] = shape.unroll;
    out[9] = shape.pairs_per_launch;
    return KVM_OK;
}

int kvm_migrate(const KvmGeom *geom, const int64_t *ctx_idx, const int64_t *dec_idx, int64_t n,
                void *dst_k, void *dst_v, int64_t dst_num_blocks, void *stream)
{
    if (n < 0) return fail(KVM_EINVAL, "n is negative");
    if (!dst_k || !dst_v) return fail(KVM_EINVAL, "destination pool is null");
    if (dst_num_blocks <= 0) return fail(KVM_EINVAL, "destination pool has no blocks");
    if (n > 0 && (!ctx_idx || !dec_idx)) return fail(KVM_EINVAL, "index list is null");
    if (n == 0) return check_geom(geom);   // an empty list moves nothing, whatever is registered
    Plan plan;
    // held until the last launch is enqueued: no registration can unmap a pool in between
    std::shared_lock<std::shared_mutex> lock(g_mu);
    if (int rc = build_plan(geom, dst_k, dst_v, &plan)) return rc;
    const uint64_t dst_bytes = (uint64_t)dst_num_blocks * plan.dst_block_stride;
    if (int rc = checked_pool(dst_k, dst_bytes, true, "decoding K pool")) return rc;
    if (int rc = checked_pool(dst_v, dst_bytes, true, "decoding V pool")) return rc;
    std::vector<IdxPair> pairs;
    bool neighbours = false;
    if (int rc = check_indices(ctx_idx, dec_idx, n, plan.min_src_blocks, dst_num_blocks,
                               "context_block_indexes", "decoding_block_indexes", &pairs, true, &neighbours))
        return rc;
    return launch_copy(std::move(plan.segs), pairs.data(), n, fits_packed(plan.min_src_blocks, dst_num_blocks),
                       (char *)dst_k, (char *)dst_v, plan.dst_block_stride, plan.vec, (hipStream_t)stream, nullptr, 0,
                       neighbours);
}

int kvm_swap_plan(const int64_t *src_ids, const int64_t *dst_ids, int64_t n, int64_t slab_bytes, int is_swap_in,
                  int64_t n_gpu_blocks, int64_t n_host_blocks, int64_t out[4])
{
    if (!out) return fail(KVM_EINVAL, "out is null");
    if (n < 0 || (n > 0 && (!src_ids || !dst_ids))) return fail(KVM_EINVAL, "bad index lists");
    if (slab_bytes <= 0 || slab_bytes >= (1ll << 32))
        return fail(KVM_EINVAL, "slab_bytes %lld must be in (0, 4 GiB)", (long long)slab_bytes);
    std::vector<IdxPair> pairs((size_t)n);
    for (int64_t i = 0; i < n; ++i) {
        if (src_ids[i] < 0 || src_ids[i] > INT32_MAX || dst_ids[i] < 0 || dst_ids[i] > INT32_MAX)
            return fail(KVM_ERANGE, "block id out of range at position %lld", (long long)i);
        pairs[(size_t)i] = IdxPair{(int32_t)src_ids[i], (int32_t)dst_ids[i]};
    }
    int64_t runs = 0;
    const int64_t mode = swap_mode_for(pairs.data(), n, slab_bytes, &runs);
    out[0] = mode;
    out[1] = runs;
    const int64_t per_launch = n_gpu_blocks > 0 && n_host_blocks > 0 && fits_packed(n_gpu_blocks, n_host_blocks) &&
                                       tune_packed() ? kMaxIdxPacked : kMaxIdx;
    out[2] = mode == 1 ? (n + per_launch - 1) / per_launch : 0;
    out[3] = mode == 1 ? (is_swap_in ? opt_swap_wgs_in.load() : opt_swap_wgs.load()) : 0;
    return KVM_OK;
}

int kvm_swap(const int64_t *src_ids, const int64_t *dst_ids, int64_t n, int is_swap_in, void *k_gpu,
             void *v_gpu, void *k_host, void *v_host, int64_t slab_bytes, int64_t n_gpu_blocks,
             int64_t n_host_blocks, void *stream)
{
    if (n < 0) return fail(KVM_EINVAL, "n is negative");
    if (!k_gpu || !v_gpu || !k_host || !v_host) return fail(KVM_EINVAL, "a pool pointer is null");
    if (slab_bytes <= 0 || slab_bytes >= (1ll << 32))
        return fail(KVM_EINVAL, "slab_bytes %lld must be in (0, 4 GiB)", (long long)slab_bytes);
    if (n_gpu_blocks <= 0 || n_host_blocks <= 0) return fail(KVM_EINVAL, "a pool has no blocks");
    if (n > 0 && (!src_ids || !dst_ids)) return fail(KVM_EINVAL, "index list is null");
    const uint64_t gpu_bytes = (uint64_t)n_gpu_blocks * (uint64_t)slab_bytes;
    const uint64_t host_bytes = (uint64_t)n_host_blocks * (uint64_t)slab_bytes;
    if (int rc = checked_pool(k_gpu, gpu_bytes, true, "GPU K pool")) return rc;
    if (int rc = checked_pool(v_gpu, gpu_bytes, true, "GPU V pool")) return rc;
    if (int rc = checked_pool(k_host, host_bytes, false, "host K pool")) return rc;
    if (int rc = checked_pool(v_host, host_bytes, false, "host V pool")) return rc;
    if (n == 0) return KVM_OK;

    const int64_t n_src = is_swap_in ? n_host_blocks : n_gpu_blocks;
    const int64_t n_dst = is_swap_in ? n_gpu_blocks : n_host_blocks;
    std::vector<IdxPair> pairs;
    if (int rc = check_indices(src_ids, dst_ids, n, n_src, n_dst, "source_block_ids", "target_block_ids",
                               &pairs))
        return rc;
    char *src_k = (char *)(is_swap_in ? k_host : k_gpu), *src_v = (char *)(is_swap_in ? v_host : v_gpu);
    char *dst_k = (char *)(is_swap_in ? k_gpu : k_host), *dst_v = (char *)(is_swap_in ? v_gpu : v_host);
    hipStream_t st = (hipStream_t)stream;

    int64_t mode = swap_mode_for(pairs.data(), n, slab_bytes, nullptr);

    // The kernel needs the pinned pools mapped into the device's address space (the default
    // for hipHostMalloc and for torch's pinned tensors).  When the choice was the library's
    // own, pools that are not mapped fall back to the copy engines; a forced mode 1 reports it.
    void *dk = nullptr, *dv = nullptr;
    if (mode == 1) {
        const hipError_t ek = hipHostGetDevicePointer(&dk, k_host, 0);
        const hipError_t ev = ek == hipSuccess ? hipHostGetDevicePointer(&dv, v_host, 0) : ek;
        if (ev != hipSuccess) {
            (void)hipGetLastError();
            if (opt_swap_mode.load() != 3)
                return fail(KVM_EHIP, "host pools are not mapped for device access: %s", hipGetErrorString(ev));
            mode = 2;
        }
    }

    if (mode == 1) {
        // One gather launch; the pinned pools are read or written in place over the host link.
        if (is_swap_in) { src_k = (char *)dk; src_v = (char *)dv; }
        else { dst_k = (char *)dk; dst_v = (char *)dv; }
        Seg s{};
        s.src_k = src_k;
        s.src_v = src_v;
        s.src_block_stride = (uint64_t)slab_bytes;
        s.src_row_stride = s.dst_row_stride = s.run_bytes = (uint32_t)slab_bytes;
        s.n_rows = 1;
        const int vec = vec_width((uint64_t)slab_bytes | (uintptr_t)src_k | (uintptr_t)src_v |
                                  (uintptr_t)dst_k | (uintptr_t)dst_v);
        return launch_copy({s}, pairs.data(), n, fits_packed(n_gpu_blocks, n_host_blocks), dst_k, dst_v,
                           (uint64_t)slab_bytes, vec, st, nullptr,
                           (int)(is_swap_in ? opt_swap_wgs_in.load() : opt_swap_wgs.load()));
    }

    // hipMemcpyAsync per run of blocks that are consecutive on both sides.  In mode 2 the V
    // pool's copies go to a second, library-owned stream forked from and joined back into
    // the caller's stream, so that two copy engines work on one call.
    const hipMemcpyKind kind = is_swap_in ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost;
    hipStream_t st_v = st;
    Fork *fork = nullptr;
    std::unique_lock<std::mutex> fork_lock;
    if (mode == 2) {
        if (int rc = get_fork(is_swap_in != 0, &fork)) return rc;
        fork_lock = std::unique_lock<std::mutex>(fork->in_use);
        KVM_HIP(hipEventRecord(fork->forked, st));
        KVM_HIP(hipStreamWaitEvent(fork->side, fork->forked, 0));
        st_v = fork->side;
    }
    int64_t i = 0;
    while (i < n) {
        int64_t j = i + 1;
        while (j < n && pairs[j].ctx == pairs[j - 1].ctx + 1 && pairs[j].dec == pairs[j - 1].dec + 1) ++j;
        const size_t bytes = (size_t)(j - i) * (size_t)slab_bytes;
        const size_t so = (size_t)pairs[i].ctx * (size_t)slab_bytes;
        const size_t dof = (size_t)pairs[i].dec * (size_t)slab_bytes;
        KVM_HIP(hipMemcpyAsync(dst_k + dof, src_k + so, bytes, kind, st));
        KVM_HIP(hipMemcpyAsync(dst_v + dof, src_v + so, bytes, kind, st_v));
        i = j;
    }
    if (fork) {
        KVM_HIP(hipEventRecord(fork->joined, fork->side));
        KVM_HIP(hipStreamWaitEvent(st, fork->joined, 0));
    }
    return KVM_OK;
}

uint32_t kvm_debug_divide(uint32_t n, uint32_t d)
{
    if (d == 0) return UINT32_MAX;
    uint32_t magic = 0, shifts = 0;
    make_magic(d, &magic, &shifts);
    // the host twin of the device's fast_div
    const uint32_t t = (uint32_t)(((uint64_t)magic * n) >> 32);
    return (t + ((n - t) >> (shifts & 0xffu))) >> (shifts >> 8);
}

int kvm_copy_plain(void *dst, const void *src, int64_t nbytes, void *stream)
{
    if (!dst || !src || nbytes < 0) return fail(KVM_EINVAL, "kvm_copy_plain: null pointer or negative size");
    if (nbytes == 0) return KVM_OK;
    if (int rc = checked_pool(dst, (uint64_t)nbytes, true, "kvm_copy_plain destination")) return rc;
    if (int rc = checked_pool(src, (uint64_t)nbytes, true, "kvm_copy_plain source")) return rc;
    // Expressed as one segment over 4 MiB "blocks" with identity index pairs; K and V
    // stand for the two halves of the buffer, as they stand for the two pools elsewhere.
    const int64_t chunk = 4ll << 20;
    const int64_t half_chunks = nbytes / (2 * chunk);
    const int vec = vec_width((uint64_t)(uintptr_t)dst | (uint64_t)(uintptr_t)src | (uint64_t)nbytes);
    int64_t done = 0;
    if (half_chunks > 0) {
        Seg s{};
        s.src_k = (const char *)src;
        s.src_v = (const char *)src + half_chunks * chunk;
        s.src_block_stride = (uint64_t)chunk;
        s.src_row_stride = s.dst_row_stride = s.run_bytes = (uint32_t)chunk;
        s.n_rows = 1;
        std::vector<IdxPair> pairs((size_t)half_chunks);
        for (int64_t i = 0; i < half_chunks; ++i) pairs[(size_t)i] = IdxPair{(int32_t)i, (int32_t)i};
        if (int rc = launch_copy({s}, pairs.data(), half_chunks, fits_packed(half_chunks, half_chunks), (char *)dst,
                                 (char *)dst + half_chunks * chunk, (uint64_t)chunk, vec, (hipStream_t)stream))
            return rc;
        done = 2 * half_chunks * chunk;
    }
    if (done < nbytes)
        KVM_HIP(hipMemcpyAsync((char *)dst + done, (const char *)src + done, (size_t)(nbytes - done),
                               hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return KVM_OK;
}

}  // extern "C"
