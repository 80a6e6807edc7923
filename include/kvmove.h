/*
 * kvmove -- C ABI of the MI355X (gfx950) KV-block migration and swap library.
 *
 * This is the drop-in boundary for the prefill->decode KV movement path of DistServe.
 * Each entry point names the reference call it stands behind (paths relative to the
 * DistServe tree).  In the reference those calls go to SwiftTransformer's
 * torch.ops.block_migration_ops.* / torch.ops.swapping_ops.swap (libst_pybinding.so);
 * here a thin torch op shim with the same schemas (distserve_amd/csrc/kvmove_torch.cpp)
 * forwards to these functions.
 *
 * Conventions
 *   - plain pointers and sizes only; no C++ or torch types cross this boundary;
 *   - every function returns KVM_OK (0) or a negative KVM_E* code and never throws;
 *     kvm_last_error() returns the calling thread's last error text;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); work is
 *     enqueued on it and the call returns without waiting for the GPU;
 *   - index arrays are read before the call returns (the caller may free them);
 *   - pools are borrowed: the caller keeps them alive while work is in flight;
 *   - calls may come from several host threads and target several streams.
 *
 * Pool layout (distserve/worker.py:107-121): contiguous
 *     [num_blocks, layers_local, kv_heads_local, block_size, head_dim]
 * K and V are separate pools of identical shape.  Pipeline rank p of P owns layers
 * [p*L/P, (p+1)*L/P) (distserve/config.py:279-286); tensor rank t of T owns KV heads
 * [t*H/T, (t+1)*H/T) (distserve/config.py:225-257).
 */
#ifndef KVMOVE_H
#define KVMOVE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KVM_OK 0
#define KVM_EINVAL (-1)     /* malformed argument (null pointer, bad size, bad geometry) */
#define KVM_ERANGE (-2)     /* a block index is outside its pool, or a pool outside its allocation */
#define KVM_EDUP (-3)       /* a destination block index occurs twice in one call */
#define KVM_ENOTREG (-4)    /* a context rank the copy needs was never registered */
#define KVM_EHIP (-5)       /* a HIP runtime call failed */
#define KVM_EHANDLE (-6)    /* memory handle is malformed, or cannot be opened in this process */
#define KVM_EMISMATCH (-7)  /* registered pools disagree with the call's geometry */

#define KVM_HANDLE_WORDS 18 /* int64 words in a memory handle */

/* Major version of this interface: kvm_version() / 10000.  It changes whenever a struct, a
 * handle or a signature below changes shape; a caller compiled against another major version
 * must not call anything but kvm_version() and kvm_last_error(). */
#define KVM_ABI_MAJOR 1

/* Device allocations of this size and above are not exported to other processes: the
 * handle of such a pool still works inside the process that made it. */
#define KVM_IPC_MAX_ALLOC_BYTES (2147483648LL)

/* Whole-model KV geometry and both instances' layouts for one migrate call.
 * The [tp_size, tp_rank, pp_size, pp_rank] order of ParallelConfig.to_list()
 * (distserve/config.py:57-63) is unpacked into named fields here. */
typedef struct KvmGeom {
    int64_t num_layers;    /* L: layers of the whole model (ModelConfig.get_num_layers()) */
    int64_t num_kv_heads;  /* H: KV heads of the whole model (ModelConfig.get_num_heads()) */
    int64_t block_size;    /* B: tokens per block (CacheConfig.block_size) */
    int64_t head_dim;      /* D */
    int64_t dtype_bytes;   /* s: 2 for fp16, 4 for fp32 (ModelConfig.get_dtype_size()) */
    int32_t ctx_pp_size;   /* context instance pipeline_parallel_size */
    int32_t ctx_tp_size;   /* context instance tensor_parallel_size */
    int32_t dec_pp_size;   /* decoding instance sizes ... */
    int32_t dec_tp_size;
    int32_t dec_pp_rank;   /* ... and the decoding rank that pulls */
    int32_t dec_tp_rank;
    int64_t ctx_instance;  /* which context instance's registered pools are read (0 = the only
                              one, as in the reference, where a decoding worker has one) */
} KvmGeom;

/* Library version: major*10000 + minor*100 + patch; the major part is KVM_ABI_MAJOR of the
 * header the library was built from. */
int kvm_version(void);

/* Text of the last error on the calling thread ("" if none). */
const char *kvm_last_error(void);

/*
 * Replaces torch.ops.block_migration_ops.get_ipc_mem_handle(tensor)
 * (distserve/worker.py:133-134).  Writes an opaque KVM_HANDLE_WORDS-word handle naming
 * the device memory [dev_ptr, dev_ptr + nbytes): the exporting process (its pid and a random
 * word it drew at start, so that two processes with one pid in different pid namespaces are
 * told apart), the pointer, and a hipIpcMemHandle_t of the device allocation that holds it
 * together with the pool's offset inside that allocation (a pool may be a piece of a larger
 * allocation, as with torch's caching allocator).  The words are plain data: send them to the decoding worker by any
 * means.  Inside the exporting process the handle resolves to the pointer itself (a
 * process cannot open its own IPC handle); in another process registration maps the
 * allocation with hipIpcOpenMemHandle.  An allocation of KVM_IPC_MAX_ALLOC_BYTES or more,
 * or one the runtime cannot export, yields a handle that is valid in its own process
 * only; another process that registers it gets KVM_EHANDLE and the reason.  The exporting
 * process must keep the allocation alive while any process uses the handle.
 */
int kvm_get_mem_handle(const void *dev_ptr, int64_t nbytes, int64_t *out_handle);

/*
 * Replaces torch.ops.block_migration_ops.register_ipc_mem_handle(k_handle, v_handle,
 * num_layers, num_heads, context_parallel_config, decoding_parallel_config)
 * (distserve/worker.py:239-246).  Binds context rank (pp_rank, tp_rank)'s K and V pools.
 * context_pc / decoding_pc are [tp_size, tp_rank, pp_size, pp_rank]
 * (distserve/config.py:57-63).  Registering the same rank again replaces the binding.
 * Handles made by another process are opened here (hipIpcOpenMemHandle, once per
 * allocation and process, however many pools lie in it) and stay mapped while a bound pool
 * lies in them (a mapping whose last pool was re-bound elsewhere is closed by the
 * registration that re-bound it, after the device has gone idle) or until kvm_reset.
 * A handle carries the exporting runtime's id of its allocation: when the exporter has
 * freed its pools and allocated new ones, handles exported afterwards replace the stale
 * mapping (and drop the pools bound through it) even where an address recurs; a handle
 * whose exporter had no id to give is mapped anew by every registration call.  A call that
 * fails leaves nothing mapped that it mapped itself.
 * ctx_instance (no counterpart in the reference, whose decoding worker serves a single
 * context instance) keeps the pools of several context instances apart in one process:
 * bindings are keyed by (ctx_instance, pp_rank, tp_rank), and a migrate call reads the
 * instance its geometry names.  Pass 0 where there is one.
 */
int kvm_register_mem_handle(const int64_t *k_handle, const int64_t *v_handle,
                            int64_t num_layers, int64_t num_kv_heads,
                            const int64_t context_pc[4], const int64_t decoding_pc[4],
                            int64_t ctx_instance);

/* Same binding from raw device pointers of this process (no handle round trip). */
int kvm_register_source(int32_t ctx_pp_size, int32_t ctx_tp_size, int32_t pp_rank, int32_t tp_rank,
                        int64_t num_layers, int64_t num_kv_heads,
                        const void *k_base, const void *v_base, int64_t nbytes_each,
                        int64_t ctx_instance);

/* Forget every registered context pool of every instance and unmap every allocation
 * opened from another process, after the device has finished the work in flight (the
 * reference has no counterpart: its registry lives as long as the worker process; tests,
 * benches and a worker that re-binds to a restarted context instance need a clean slate). */
int kvm_reset(void);

/* Allocations of other processes currently mapped by registration (for tests and reports). */
int64_t kvm_opened_handles(void);

/*
 * Replaces torch.ops.block_migration_ops.migrate_blocks(...)
 * (distserve/worker.py:250-267).  For i in [0, n), X in {K, V} and every (layer l,
 * kv head h) of decoding rank (dec_pp_rank, dec_tp_rank):
 *     dstX[dec_idx[i], l - l0_dec, h - h0_dec, :, :] =
 *         srcX{owner(l,h)}[ctx_idx[i], l - l0_ctx, h - h0_ctx, :, :]
 * Source pools are the registered ones; they are only read.  Destination blocks not
 * named in dec_idx are not touched.  dec_idx must not repeat a block (KVM_EDUP);
 * ctx_idx may.  n == 0 is a no-op.
 */
int kvm_migrate(const KvmGeom *geom, const int64_t *ctx_idx, const int64_t *dec_idx, int64_t n,
                void *dst_k, void *dst_v, int64_t dst_num_blocks, void *stream);

/*
 * Replaces torch.ops.swapping_ops.swap(source_block_ids, target_block_ids, is_swap_in,
 * k_cache, v_cache, k_swap, v_swap) (distserve/worker.py:303-311).
 * is_swap_in != 0:  gpuX[dst_ids[i]]  = hostX[src_ids[i]]
 * is_swap_in == 0:  hostX[dst_ids[i]] = gpuX[src_ids[i]]        for X in {K, V}.
 * slab_bytes is one block of one pool (layers_local*heads_local*B*D*s).  Host pools
 * must be pinned (hipHostMalloc / torch pin_memory) for the copy to be asynchronous.
 * dst_ids must not repeat a block.
 */
int kvm_swap(const int64_t *src_ids, const int64_t *dst_ids, int64_t n, int is_swap_in,
             void *k_gpu, void *v_gpu, void *k_host, void *v_host, int64_t slab_bytes,
             int64_t n_gpu_blocks, int64_t n_host_blocks, void *stream);

/*
 * Plain contiguous device copy with the same load/store code as the migration kernel.
 * No counterpart in the reference: it calibrates hardware counters (a copy of known
 * size) and gives the attainable streaming-copy ceiling beside the migration figure.
 */
int kvm_copy_plain(void *dst, const void *src, int64_t nbytes, void *stream);

/*
 * Options (no counterpart in the reference), process-wide.  Names:
 *   "xcd_map"        how workgroup ids map to work: 0 = in order, 1 (default) = chosen per call:
 *                    in order when at least half of the call's context blocks follow their
 *                    predecessor in the list directly (neighbouring blocks), else each XCD walks
 *                    contiguous chunks (an eighth of a block when that is >= 256 KiB, else an
 *                    eighth of the launch), 2 = always an eighth of the launch, 3 = always an
 *                    eighth of a block
 *   "sort_pairs"     order in which a migrate call's (context block, decoding block) pairs reach
 *                    the kernel; the copy does not depend on it, the memory system does.
 *                    1 (default) = by context block when the call names at least a quarter of
 *                    the context pool (then most of the pool is read front to back: +4 % on
 *                    calls of 800 of 1024 blocks whose rows are half read), else the caller's
 *                    order; 0 = always the caller's order; 2 = always by context block
 *   "swap_mode"      3 (default) = chosen per call: mode 1, unless the copies of the call average
 *                        "swap_kernel_below" bytes or more each or the pinned pools are not mapped
 *                        for device access, then mode 2,
 *                    1 = copy kernel that reads/writes the pinned pools in place: one launch
 *                        per 864 blocks whatever their size, about 0.1 ms of host time for 2048
 *                        blocks, 97-100 % of the link,
 *                    2 = hipMemcpyAsync per run of blocks consecutive on both sides, K pool on
 *                        the caller's stream and V pool on a second stream forked from and
 *                        joined back into it: two runtime calls per block (4-5 ms of host time
 *                        for 2048 blocks), 97-98 % of the link for copies of 4 MiB, less below,
 *                    0 = the same with both pools on the caller's stream (87 %)
 *   "swap_wgs"       workgroups per pool kind of the swap kernel for a swap-out, 1..4096; a
 *                    workgroup keeps 4 KiB in flight.  Default 16: 99 % of the link on an idle GPU,
 *                    97 % while other kernels saturate HBM, and a migration beside it 2-3 % slower
 *   "swap_wgs_in"    the same for a swap-in.  Default 16: 99 % idle, 85 % beside kernels that
 *                    saturate HBM, a migration beside it 2-3 % slower; with a swap-out and a swap-in
 *                    in flight together, 46 GB/s each way (two large copies both ways: 49-52 down,
 *                    30-57 up).  The trade is between the swap's share of the link while HBM is
 *                    saturated and what the kernels beside it lose: 18 workgroups 94 % and 3.5 %,
 *                    20: 96 % and 4 %, 36: 98 % and 15 %, 64 and more: several times slower
 *   "swap_kernel_below"  bytes per copy under which mode 3 takes the kernel (default 4 GiB, i.e.
 *                    always; 2 MiB hands large slabs to the copy engines)
 * A library built with -DKVM_EXPLORE (sweeps and the tests that show every kernel flavour
 * copies the same bytes; never shipped) knows more names: the workgroup shape, cache
 * policy and tile size of the copy kernel.
 * kvm_get_option returns the value or KVM_EINVAL (as int64) for an unknown name.
 */
int kvm_set_option(const char *name, int64_t value);
int64_t kvm_get_option(const char *name);

/*
 * Launch shape kvm_migrate would use for this geometry and n blocks, for tests and
 * reports: out[0] = workgroups per block (K and V together), out[1] = workgroup size,
 * out[2] = vector width in bytes, out[3] = number of source segments,
 * out[4] = kernel launches, out[5] = payload bytes per block (K+V, this rank's share),
 * out[6] = 1 when the short-prologue kernel (kvm_copy_simple_kernel) serves the shape,
 * out[7] = work-items (workgroups x workgroup size) of the largest launch, which the
 * library keeps below 2^32 by splitting the block list over more launches,
 * out[8] = 16-byte vectors each lane moves, out[9] = index pairs one launch carries at most
 * (864 when the context pools and a destination pool of dst_num_blocks blocks all have at
 * most 65536 blocks, so that a pair packs into 32 bits; else 432; fewer for huge blocks).
 * dst_num_blocks <= 0 = unknown (plans for 432).
 * Needs the sources registered (alignment of their bases picks the vector width), except
 * with dst_k == dst_v == NULL: then the plan is pure arithmetic, touches no device, takes
 * every pool for 16-byte aligned and the context pools for dst_num_blocks blocks each.
 */
int kvm_migrate_plan(const KvmGeom *geom, int64_t n, const void *dst_k, const void *dst_v,
                     int64_t dst_num_blocks, int64_t out[10]);

/*
 * How kvm_swap would serve these lists at this slab size under the current options, for
 * tests and reports (no counterpart in the reference): out[0] = implementation taken (0, 1
 * or 2, as "swap_mode" numbers them), out[1] = copies per pool = runs of blocks consecutive
 * on both sides, out[2] = kernel launches (mode 1, else 0), out[3] = workgroups per pool
 * kind of each launch (mode 1, else 0; swap-in and swap-out have their own counts).
 * n_gpu_blocks / n_host_blocks: the pools' sizes, which decide how many blocks one launch
 * carries (864 when both are at most 65536, else 432; <= 0 = unknown, plans for 432).  Touches
 * no device and no pool (so it cannot see whether pinned pools are mapped for the kernel).
 */
int kvm_swap_plan(const int64_t *src_ids, const int64_t *dst_ids, int64_t n, int64_t slab_bytes,
                  int is_swap_in, int64_t n_gpu_blocks, int64_t n_host_blocks, int64_t out[4]);

/*
 * Test hook (no counterpart in the reference): n / d computed the way the kernel computes
 * a tile's row, with the multiplier and shifts the host derives for d.  Lets a CPU test
 * check that arithmetic against plain division.  Returns UINT32_MAX for d == 0.
 */
uint32_t kvm_debug_divide(uint32_t n, uint32_t d);

#ifdef __cplusplus
}
#endif
#endif /* KVMOVE_H */
