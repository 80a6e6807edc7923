// What the memory system of one MI355X delivers for the address patterns of the KV copy,
// measured with the plainest kernels that can produce them.  Not part of the library: a
// stand-alone program that answers "how fast could ANY kernel move these bytes", so that
// the migration kernels' figures can be read against a measured ceiling instead of the
// data-sheet one.
//
//   hbm_probe [--quick] [--section 1|2|3]
//
// Every kernel is "one shot": a workgroup handles one tile (lanes x vectors x 16 bytes)
// and ends, the form the migration kernels use.  Tile t of a launch reads
//     src + (t / run_tiles) * src_stride + (t % run_tiles) * tile_bytes
// and writes dst + t * tile_bytes, so (run, stride) = (8 KiB, 16 KiB) is the source pattern
// of a decoding rank that wants two of a context rank's four heads, and run == stride is a
// dense stream.  There are no index tables, no segments and no division: addresses come
// from shifts of the workgroup id (sections 1 and 2 of the output; the sources can also be
// regions scattered over the buffer).  Section 3 adds what sections 1 and 2 leave out of the
// real copy, block tables and the pools' geometry, in the plainest form: table_kernel below,
// with the geometry in template constants.  Launches rotate over windows of the buffers, or
// draw fresh block lists, so that no launch finds its bytes in the 256 MB last-level cache.
//
// Build: make -C tests/hbm_probe (hipcc --offload-arch=gfx950 -O3 hbm_probe.hip -o hbm_probe).

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CHECK(expr)                                                                              \
    do {                                                                                         \
        hipError_t e_ = (expr);                                                                  \
        if (e_ != hipSuccess) {                                                                  \
            fprintf(stderr, "%s:%d: %s failed: %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
            exit(2);                                                                             \
        }                                                                                        \
    } while (0)

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define GLOBAL_AS __attribute__((address_space(1)))

enum Mode { kRead = 0, kWrite = 1, kCopy = 2 };

struct ProbeArgs {
    char *dst;
    const char *src;
    uint32_t tiles;           // tiles of this launch
    uint32_t run_shift;       // log2(tiles per source run)
    uint64_t src_stride;      // bytes from one source run to the next
    uint32_t chunk_shift;     // log2(tiles one XCD takes at a time); 31 = workgroup ids in order
    // scattered sources: the launch's tiles form regions of 2^region_shift tiles, and region r is
    // read from place ((r + region_base) * odd) mod 2^k of the source buffer (31 = no regions)
    uint32_t region_shift;
    uint32_t region_base, region_mask;
    uint64_t region_span;     // bytes of source buffer one region occupies
};

// id -> tile: ids are dealt round-robin to the 8 XCDs; with chunk_shift < 31 each XCD walks
// contiguous chunks of tiles (the mapping of the migration kernels, with shifts).
__device__ __forceinline__ uint32_t tile_of(uint32_t id, uint32_t chunk_shift)
{
    if (chunk_shift >= 31) return id;
    const uint32_t xcd = id & 7u, seq = id >> 3;
    const uint32_t q = seq >> chunk_shift;
    return ((q * 8u + xcd) << chunk_shift) + (seq & ((1u << chunk_shift) - 1u));
}

template <int MODE, int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void probe_kernel(const ProbeArgs a)
{
    constexpr uint32_t kTile = THREADS * UNROLL * 16u;
    const uint32_t t = tile_of(blockIdx.x, a.chunk_shift);
    if (t >= a.tiles) return;
    uint32_t ts = t;          // the tile's place in the source pattern
    uint64_t soff = 0;
    if (a.region_shift < 31) {
        const uint32_t region = ((t >> a.region_shift) + a.region_base) * 0x9E3779B1u & a.region_mask;
        soff = (uint64_t)region * a.region_span;
        ts = t & ((1u << a.region_shift) - 1u);
    }
    const uint32_t run = ts >> a.run_shift, within = ts & ((1u << a.run_shift) - 1u);
    soff += (uint64_t)run * a.src_stride + (uint64_t)within * kTile;
    const uint64_t doff = (uint64_t)t * kTile;
    u32x4 r[UNROLL];
    if constexpr (MODE != kWrite) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const GLOBAL_AS u32x4 *p = reinterpret_cast<const GLOBAL_AS u32x4 *>(
                (uint64_t)a.src + soff + (uint64_t)(u * THREADS + threadIdx.x) * 16u);
            r[u] = __builtin_nontemporal_load(p);
        }
    } else {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) r[u] = u32x4{t, (uint32_t)u, threadIdx.x, 0u};
    }
    if constexpr (MODE != kRead) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            GLOBAL_AS u32x4 *p = reinterpret_cast<GLOBAL_AS u32x4 *>(
                (uint64_t)a.dst + doff + (uint64_t)(u * THREADS + threadIdx.x) * 16u);
            asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(r[u]) : "memory");
        }
    } else {
        // the loaded registers must be awaited, or the wave would end with its loads unissued
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) asm volatile("" : : "v"(r[u]));
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
}

// The copy with block tables, at a fixed geometry and nothing else: block b of the launch is
// NSEG segments of ROWS rows of ROW_TILES one-KiB tiles; segment j of it is read from block
// src_ids[b] of source pool j, where a row starts every ROW_STRIDE_TILES KiB, and the block
// is written densely to block dst_ids[b] of the destination pool.  <8, 16, 40, 2, false> is
// one pool kind of a request of the 70B configuration (two of four heads from each of two
// pipeline stages); <8, 8, 40, 2, false> is the same bytes from pools that hold exactly
// those two heads; <80, 80, 40, 2, true> is the 13B configuration (each of 40 layer rows is
// 80 KiB from each of two tensor-parallel ranks, side by side).
struct TableArgs {
    char *dst;
    const char *src[2];
    const int32_t *src_ids, *dst_ids;
    uint32_t tiles, chunk_tiles;   // chunk_tiles 0 = workgroup ids in order
    uint32_t src_row_off;          // bytes into a source row where the wanted bytes start
    uint32_t pad;
};

template <int ROW_TILES, int ROW_STRIDE_TILES, int ROWS, int NSEG, bool INTERLEAVED>
__global__ __launch_bounds__(64) void table_kernel(const TableArgs a)
{
    constexpr uint32_t kBlockTiles = ROW_TILES * ROWS * NSEG, kSegTiles = ROW_TILES * ROWS;
    uint32_t t = blockIdx.x;
    if (a.chunk_tiles != 0) {
        const uint32_t xcd = t & 7u, seq = t >> 3;
        const uint32_t q = seq / a.chunk_tiles;
        t = (q * 8u + xcd) * a.chunk_tiles + (seq - q * a.chunk_tiles);
    }
    if (t >= a.tiles) return;
    // u: the tile's place in the destination block, which is written densely
    const uint32_t b = t / kBlockTiles, u = t - b * kBlockTiles;
    uint32_t seg, row, within;
    if constexpr (INTERLEAVED) {   // a destination row is the segments' rows side by side
        row = u / (ROW_TILES * NSEG);
        const uint32_t v = u - row * (ROW_TILES * NSEG);
        seg = v / ROW_TILES;
        within = v - seg * ROW_TILES;
    } else {                       // the segments follow each other
        seg = u / kSegTiles;
        const uint32_t v = u - seg * kSegTiles;
        row = v / ROW_TILES;
        within = v - row * ROW_TILES;
    }
    const uint64_t sblock = (uint64_t)(uint32_t)a.src_ids[b] * (ROW_STRIDE_TILES * ROWS * 1024u);
    const uint64_t dblock = (uint64_t)(uint32_t)a.dst_ids[b] * (kBlockTiles * 1024u);
    const uint64_t saddr = (uint64_t)a.src[seg] + sblock + row * (ROW_STRIDE_TILES * 1024u) + a.src_row_off +
                           within * 1024u + threadIdx.x * 16u;
    const uint64_t daddr = (uint64_t)a.dst + dblock + u * 1024u + threadIdx.x * 16u;
    const u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const GLOBAL_AS u32x4 *>(saddr));
    GLOBAL_AS u32x4 *p = reinterpret_cast<GLOBAL_AS u32x4 *>(daddr);
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(r) : "memory");
}

struct Flavour {
    const char *name;
    int threads, unroll;
    void (*fn[3])(const ProbeArgs);
};

#define FLAVOUR(T, U) {#T "x" #U, T, U, {probe_kernel<kRead, T, U>, probe_kernel<kWrite, T, U>, probe_kernel<kCopy, T, U>}}
static const Flavour kFlavours[] = {FLAVOUR(64, 1), FLAVOUR(64, 2), FLAVOUR(256, 1), FLAVOUR(256, 4)};

static uint32_t log2_exact(uint64_t v, const char *what)
{
    uint32_t s = 0;
    while ((1ull << s) < v) ++s;
    if ((1ull << s) != v) {
        fprintf(stderr, "%s = %llu is not a power of two\n", what, (unsigned long long)v);
        exit(2);
    }
    return s;
}

struct Result {
    double us_per_launch, gbps;
};

// `launches` launches of `bytes` algorithmic bytes each way, back to back on the null stream,
// each over its own window of the buffers; HIP events around all of them.
static Result run_case(const Flavour &f, Mode mode, char *dst, const char *src, uint64_t buf_bytes, uint64_t bytes,
                       uint64_t run_bytes, uint64_t stride_bytes, uint64_t chunk_bytes, uint64_t region_bytes,
                       int launches)
{
    const uint64_t tile = (uint64_t)f.threads * f.unroll * 16u;
    const uint64_t tiles = bytes / tile;
    const uint64_t src_span = bytes / run_bytes * stride_bytes;
    const uint64_t windows = std::max<uint64_t>(1, std::min(buf_bytes / src_span, buf_bytes / bytes));
    if (src_span > buf_bytes || tiles >= (1ull << 31) / 8 * 8 || tiles * (uint64_t)f.threads >= (1ull << 32)) {
        fprintf(stderr, "case does not fit: %llu bytes over a span of %llu\n", (unsigned long long)bytes,
                (unsigned long long)src_span);
        exit(2);
    }
    ProbeArgs a{};
    a.tiles = (uint32_t)tiles;
    a.run_shift = log2_exact(run_bytes / tile, "tiles per run");
    a.src_stride = stride_bytes;
    a.chunk_shift = chunk_bytes ? log2_exact(chunk_bytes / tile, "tiles per chunk") : 31;
    a.region_shift = 31;
    uint32_t regions_per_launch = 0;
    if (region_bytes) {
        a.region_shift = log2_exact(region_bytes / tile, "tiles per region");
        a.region_span = region_bytes / run_bytes * stride_bytes;
        a.region_mask = (uint32_t)(buf_bytes / a.region_span) - 1u;
        log2_exact((uint64_t)a.region_mask + 1, "regions in the buffer");
        regions_per_launch = (uint32_t)(bytes / region_bytes);
    }
    uint64_t grid = tiles;
    if (chunk_bytes) {
        const uint64_t per_round = 8ull << a.chunk_shift;
        grid = (tiles + per_round - 1) / per_round * per_round;
    }
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    float total = 0;
    const int passes = 3;
    for (int pass = 0; pass < passes + 1; ++pass) {   // the first pass warms up
        CHECK(hipEventRecord(e0, nullptr));
        for (int l = 0; l < launches; ++l) {
            const uint64_t w = (uint64_t)(pass * launches + l) % windows;
            a.src = region_bytes ? src : src + w * src_span;
            a.region_base = (uint32_t)(pass * launches + l) * regions_per_launch;
            a.dst = dst + w * bytes;
            hipLaunchKernelGGL(f.fn[mode], dim3((uint32_t)grid), dim3(f.threads), 0, nullptr, a);
        }
        CHECK(hipEventRecord(e1, nullptr));
        CHECK(hipEventSynchronize(e1));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        if (pass > 0) total += ms;
    }
    CHECK(hipGetLastError());
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    const double us = (double)total / passes / launches * 1e3;
    const double traffic = (mode == kCopy ? 2.0 : 1.0) * (double)bytes;
    return Result{us, traffic / (us * 1e-6) / 1e9};
}

// Block-table copies: `launches` launches of `nb` blocks each, lists sequential (advancing
// through the pools) or random (no block twice in a launch), back to back.  src_order 2:
// random picks, in ascending order of the source block (the destination blocks keep the
// random order they were drawn in): what a call's pairs look like once sorted by source.
template <int ROW_TILES, int ROW_STRIDE_TILES, int ROWS, int NSEG, bool INTERLEAVED>
static Result run_table(char *dst, const char *src, uint32_t src_blocks, uint32_t dst_blocks, uint32_t nb,
                        int src_order, bool dst_random, int chunk_mode, int launches)
{
    constexpr uint32_t kBlockTiles = ROW_TILES * ROWS * NSEG;
    const int passes = 3, total_launches = (passes + 1) * launches;
    std::vector<int32_t> sid((size_t)total_launches * nb), did((size_t)total_launches * nb);
    uint64_t rng = 0x243F6A8885A308D3ull;
    auto next = [&rng]() {
        rng = rng * 6364136223846793005ull + 1442695040888963407ull;
        return (uint32_t)(rng >> 33);
    };
    auto fill = [&](std::vector<int32_t> &ids, uint32_t pool_blocks, int order) {
        std::vector<int32_t> perm(pool_blocks);
        uint32_t off = 0;
        for (int l = 0; l < total_launches; ++l) {
            for (uint32_t i = 0; i < pool_blocks; ++i) perm[i] = (int32_t)((off + i) % pool_blocks);
            if (order != 0)
                for (uint32_t i = 0; i < nb; ++i) std::swap(perm[i], perm[i + next() % (pool_blocks - i)]);
            if (order == 2) std::sort(perm.begin(), perm.begin() + nb);
            for (uint32_t i = 0; i < nb; ++i) ids[(size_t)l * nb + i] = perm[i];
            off += nb;
        }
    };
    fill(sid, src_blocks, src_order);
    fill(did, dst_blocks, dst_random ? 1 : 0);
    int32_t *d_sid = nullptr, *d_did = nullptr;
    CHECK(hipMalloc((void **)&d_sid, sid.size() * 4));
    CHECK(hipMalloc((void **)&d_did, did.size() * 4));
    CHECK(hipMemcpy(d_sid, sid.data(), sid.size() * 4, hipMemcpyHostToDevice));
    CHECK(hipMemcpy(d_did, did.data(), did.size() * 4, hipMemcpyHostToDevice));

    TableArgs a{};
    a.dst = dst;
    a.src[0] = src;
    a.src[1] = src + (4ull << 30);
    if ((uint64_t)src_blocks * ROW_STRIDE_TILES * ROWS * 1024u > (4ull << 30) ||
        (uint64_t)dst_blocks * kBlockTiles * 1024u > (8ull << 30) || nb > src_blocks || nb > dst_blocks ||
        (uint64_t)nb * kBlockTiles * 64u >= (1ull << 32)) {
        fprintf(stderr, "table case does not fit the buffers or the grid\n");
        exit(2);
    }
    a.tiles = nb * kBlockTiles;
    a.chunk_tiles = chunk_mode == 0 ? 0 : chunk_mode == 1 ? (a.tiles + 7) / 8 : 256;
    a.src_row_off = (ROW_STRIDE_TILES - ROW_TILES) * 1024u;   // the wanted heads are the last of the row
    uint32_t grid = a.tiles;
    if (a.chunk_tiles) grid = (a.tiles + 8 * a.chunk_tiles - 1) / (8 * a.chunk_tiles) * (8 * a.chunk_tiles);
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    float total = 0;
    for (int pass = 0; pass < passes + 1; ++pass) {
        CHECK(hipEventRecord(e0, nullptr));
        for (int l = 0; l < launches; ++l) {
            a.src_ids = d_sid + (size_t)(pass * launches + l) * nb;
            a.dst_ids = d_did + (size_t)(pass * launches + l) * nb;
            hipLaunchKernelGGL((table_kernel<ROW_TILES, ROW_STRIDE_TILES, ROWS, NSEG, INTERLEAVED>), dim3(grid), dim3(64), 0, nullptr, a);
        }
        CHECK(hipEventRecord(e1, nullptr));
        CHECK(hipEventSynchronize(e1));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        if (pass > 0) total += ms;
    }
    CHECK(hipGetLastError());
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    CHECK(hipFree(d_sid));
    CHECK(hipFree(d_did));
    const double us = (double)total / passes / launches * 1e3;
    return Result{us, 2.0 * a.tiles * 1024.0 / (us * 1e-6) / 1e9};
}

int main(int argc, char **argv)
{
    bool quick = false;
    int only = 0;   // 0 = every section
    for (int i = 1; i < argc; ++i) {
        if (!strcmp(argv[i], "--quick")) quick = true;
        else if (!strcmp(argv[i], "--section") && i + 1 < argc && atoi(argv[i + 1]) >= 1 && atoi(argv[i + 1]) <= 3)
            only = atoi(argv[++i]);
        else {
            fprintf(stderr, "usage: hbm_probe [--quick] [--section 1|2|3]\n"
                            "  --quick      sections 1 and 2 with 64 lanes x 1 vector only\n"
                            "  --section N  only section N (1 one-way streams, 2 strided copies, 3 block tables)\n");
            return 2;
        }
    }
    CHECK(hipSetDevice(0));
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const uint64_t kBuf = 8ull << 30;   // per buffer: many windows even for the long launches
    char *src = nullptr, *dst = nullptr;
    CHECK(hipMalloc((void **)&src, kBuf));
    CHECK(hipMalloc((void **)&dst, kBuf));
    CHECK(hipMemset(src, 0x5a, kBuf));
    CHECK(hipMemset(dst, 0, kBuf));
    CHECK(hipDeviceSynchronize());
    printf("hbm_probe on %s (%d CUs): one-shot kernels, nontemporal 16-byte loads, sc1 nt stores\n", prop.name,
           prop.multiProcessorCount);
    printf("GB/s counts bytes read + bytes written (a copy counts both); MI355X data sheet: 8000 GB/s\n\n");

    struct Pattern {
        const char *name;
        uint64_t run, stride;
    };
    const Pattern patterns[] = {
        {"dense", 64 << 10, 64 << 10},
        {"8 KiB on / 8 KiB off", 8 << 10, 16 << 10},
        {"8 KiB on / 24 KiB off", 8 << 10, 32 << 10},
        {"64 KiB on / 64 KiB off", 64 << 10, 128 << 10},
    };
    struct Size {
        const char *name;
        uint64_t bytes;
        int launches;
    };
    // 160 MiB each way is what one request of the 70B configuration moves on average
    // (136.5 blocks x 1.25 MiB); 1 GiB is a launch long enough that ramp and tail vanish.
    const Size sizes[] = {{"160 MiB", 160ull << 20, 24}, {"1 GiB", 1ull << 30, 6}};
    const uint64_t chunks[] = {0, 256 << 10};
    // where the source's bytes lie: one contiguous window, or regions of this many wanted
    // bytes scattered over the 8 GiB buffer (a KV block of a pool is such a region)
    const uint64_t regions[] = {0, 256 << 10, 4 << 20};
    const char *region_name[] = {"contiguous", "256 KiB scattered", "4 MiB scattered"};
    const char *mode_name[] = {"read", "write", "copy"};

    printf("1. One-way streams, dense\n");
    printf("%-8s %-6s %-10s %-10s %12s %10s\n", "lanes x", "mode", "bytes per", "workgroup", "us/launch", "GB/s");
    printf("%-8s %-6s %-10s %-10s\n", "vectors", "", "launch", "ids");
    for (const Flavour &f : kFlavours) {
        if (only && only != 1) break;
        if (quick && !(f.threads == 64 && f.unroll == 1)) continue;
        for (int mode = 0; mode < 2; ++mode) {
            for (const Size &s : sizes) {
                for (uint64_t chunk : chunks) {
                    const Result r = run_case(f, (Mode)mode, dst, src, kBuf, s.bytes, patterns[0].run,
                                              patterns[0].stride, chunk, 0, s.launches);
                    printf("%-8s %-6s %-10s %-10s %12.2f %10.1f\n", f.name, mode_name[mode], s.name,
                           chunk ? "256K/XCD" : "in order", r.us_per_launch, r.gbps);
                    fflush(stdout);
                }
            }
        }
    }

    printf("\n2. Copies into a dense destination\n");
    printf("%-8s %-24s %-18s %-10s %-10s %12s %10s\n", "lanes x", "source pattern", "source placement", "bytes per",
           "workgroup", "us/launch", "GB/s");
    printf("%-8s %-24s %-18s %-10s %-10s\n", "vectors", "", "", "launch", "ids");
    for (const Flavour &f : kFlavours) {
        const bool migration_shape = f.threads == 64 && f.unroll == 1;
        if (only && only != 2) break;
        if (quick && !migration_shape) continue;
        for (const Pattern &p : patterns) {
            const uint64_t tile = (uint64_t)f.threads * f.unroll * 16u;
            if (p.run < tile) continue;
            if (!migration_shape && f.unroll != 1 && p.run != p.stride) continue;   // other shapes: dense only
            for (int g = 0; g < 3; ++g) {
                if (!migration_shape && f.unroll != 1 && g != 0) continue;
                for (const Size &s : sizes) {
                    for (uint64_t chunk : chunks) {
                        const Result r = run_case(f, kCopy, dst, src, kBuf, s.bytes, p.run, p.stride, chunk, regions[g],
                                                  s.launches);
                        printf("%-8s %-24s %-18s %-10s %-10s %12.2f %10.1f\n", f.name, p.name, region_name[g], s.name,
                               chunk ? "256K/XCD" : "in order", r.us_per_launch, r.gbps);
                        fflush(stdout);
                    }
                }
            }
        }
    }
    printf("\n3. Copies through block tables (64 lanes x 1 vector; block ids from tables in device memory)\n"
           "   70B: blocks of 2 segments x 40 rows x 8 KiB, one segment after the other; 1024-block source pools, 2048-block\n"
           "        destination pool.  13B: blocks of 40 rows x (80 KiB from each of 2 pools); 1024-block pools.\n");
    printf("%-22s %-8s %-8s %-10s %-12s %12s %10s\n", "source rows", "source", "dest.", "blocks per", "workgroup", "us/launch",
           "GB/s");
    printf("%-22s %-8s %-8s %-10s %-12s\n", "", "blocks", "blocks", "launch", "ids");
    const char *chunk_name[] = {"in order", "launch/8", "256K/XCD"};
    const char *geom_name[] = {"70B 8 KiB of 16 KiB", "70B 8 KiB of 8 KiB", "13B 2 x 80 KiB"};
    for (int geom = 0; geom < 3; ++geom) {
        if (only && only != 3) break;
        // per-request and long launches: 272 / 1024 blocks of 640 KiB, 72 / 864 blocks of 6.25 MiB
        const uint32_t nbs[2] = {geom == 2 ? 72u : 272u, geom == 2 ? 864u : 1024u};
        for (int size = 0; size < 2; ++size) {
            for (int sr = 0; sr < 2; ++sr) {
                for (int dr = 0; dr < 2; ++dr) {
                    for (int cm = 0; cm < 3; ++cm) {
                        const uint32_t nb = nbs[size];
                        const int launches = size == 0 ? 24 : geom == 2 ? 3 : 6;
                        const Result r =
                            geom == 0   ? run_table<8, 16, 40, 2, false>(dst, src, 1024, 2048, nb, sr, dr, cm, launches)
                            : geom == 1 ? run_table<8, 8, 40, 2, false>(dst, src, 1024, 2048, nb, sr, dr, cm, launches)
                                        : run_table<80, 80, 40, 2, true>(dst, src, 1024, 1024, nb, sr, dr, cm, launches);
                        printf("%-22s %-8s %-8s %-10u %-12s %12.2f %10.1f\n", geom_name[geom], sr ? "random" : "adjacent",
                               dr ? "random" : "adjacent", nb, chunk_name[cm], r.us_per_launch, r.gbps);
                        fflush(stdout);
                    }
                }
            }
        }
    }
    // A call that names most of the source pool: its random picks in the order drawn, and
    // sorted by source block (with ids in order, most of the pool is then read front to back).
    for (uint32_t nb : {272u, 800u}) {
        if (only && only != 3) break;
        for (int sr = 1; sr <= 2; ++sr) {
            for (int cm = 0; cm < 3; ++cm) {
                const Result r = run_table<8, 16, 40, 2, false>(dst, src, 1024, 2048, nb, sr, true, cm, nb == 272 ? 24 : 6);
                printf("%-22s %-8s %-8s %-10u %-12s %12.2f %10.1f\n", geom_name[0], sr == 1 ? "random" : "sorted", "random",
                       nb, chunk_name[cm], r.us_per_launch, r.gbps);
                fflush(stdout);
            }
        }
    }
    CHECK(hipFree(src));
    CHECK(hipFree(dst));
    return 0;
}
