// kvmove_torch.cpp -- torch op shim over the kvmove C ABI.
//
// Registers the four ops DistServe's worker looks up after torch.ops.load_library
// (distserve/__init__.py:16), with the argument order of their call sites:
//   block_migration_ops::get_ipc_mem_handle        distserve/worker.py:133-134
//   block_migration_ops::register_ipc_mem_handle   distserve/worker.py:239-246
//   block_migration_ops::migrate_blocks            distserve/worker.py:256-267
//   swapping_ops::swap                             distserve/worker.py:303-311
// No data is touched here: tensors are checked, reduced to pointers and sizes, and the
// current HIP stream is handed to the C ABI.  A nonzero return code becomes a
// RuntimeError carrying kvm_last_error().
#include "kvmove.h"

#include <c10/hip/HIPStream.h>
#include <torch/library.h>
#include <ATen/ATen.h>

#include <vector>

namespace {

void check(int rc, const char *op)
{
    TORCH_CHECK(rc == KVM_OK, op, ": ", kvm_last_error(), " (kvmove error ", rc, ")");
}

void check_pool(const at::Tensor &t, const char *name, bool on_gpu)
{
    TORCH_CHECK(t.dim() == 5, name, " must be [num_blocks, layers, kv_heads, block_size, head_dim], got ",
                t.dim(), " dims");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    if (on_gpu) {
        TORCH_CHECK(t.is_cuda(), name, " must live on the GPU");
    } else {
        TORCH_CHECK(t.is_cpu() && t.is_pinned(), name, " must be pinned host memory");
    }
}

void *current_stream(const at::Tensor &on)
{
    return (void *)c10::hip::getCurrentHIPStream(on.device().index()).stream();
}

std::vector<int64_t> get_ipc_mem_handle(const at::Tensor &t)
{
    TORCH_CHECK(t.is_cuda() && t.is_contiguous(), "get_ipc_mem_handle wants a contiguous GPU tensor");
    std::vector<int64_t> h(KVM_HANDLE_WORDS);
    check(kvm_get_mem_handle(t.data_ptr(), (int64_t)t.nbytes(), h.data()), "get_ipc_mem_handle");
    return h;
}

// The *_from forms (no counterpart in the reference) name the context instance whose pools
// are bound or read, for a process that serves more than one; the reference's own schemas
// below them mean instance 0.
void register_ipc_mem_handle_from(int64_t context_instance, std::vector<int64_t> k_handle,
                                  std::vector<int64_t> v_handle, int64_t num_layers, int64_t num_heads,
                                  std::vector<int64_t> context_parallel_config,
                                  std::vector<int64_t> decoding_parallel_config)
{
    TORCH_CHECK(k_handle.size() == KVM_HANDLE_WORDS && v_handle.size() == KVM_HANDLE_WORDS,
                "register_ipc_mem_handle: a memory handle has ", KVM_HANDLE_WORDS, " words");
    TORCH_CHECK(context_parallel_config.size() == 4 && decoding_parallel_config.size() == 4,
                "register_ipc_mem_handle: parallel configs are [tp_size, tp_rank, pp_size, pp_rank]");
    check(kvm_register_mem_handle(k_handle.data(), v_handle.data(), num_layers, num_heads,
                                  context_parallel_config.data(), decoding_parallel_config.data(),
                                  context_instance),
          "register_ipc_mem_handle");
}

void register_ipc_mem_handle(std::vector<int64_t> k_handle, std::vector<int64_t> v_handle,
                             int64_t num_layers, int64_t num_heads,
                             std::vector<int64_t> context_parallel_config,
                             std::vector<int64_t> decoding_parallel_config)
{
    register_ipc_mem_handle_from(0, std::move(k_handle), std::move(v_handle), num_layers, num_heads,
                                 std::move(context_parallel_config), std::move(decoding_parallel_config));
}

void migrate_blocks_from(int64_t context_instance, int64_t context_pp_size, int64_t context_tp_size,
                         std::vector<int64_t> context_block_indexes, int64_t decoding_pp_size,
                         int64_t decoding_tp_size, int64_t decoding_pp_rank, int64_t decoding_tp_rank,
                         std::vector<int64_t> decoding_block_indexes, const at::Tensor &k_cache,
                         const at::Tensor &v_cache)
{
    check_pool(k_cache, "k_cache", true);
    check_pool(v_cache, "v_cache", true);
    TORCH_CHECK(k_cache.sizes() == v_cache.sizes() && k_cache.dtype() == v_cache.dtype() &&
                    k_cache.device() == v_cache.device(),
                "k_cache and v_cache must agree in shape, dtype and device");
    // the engine asserts this before the call (distserve/single_stage_engine.py:517)
    TORCH_CHECK(context_block_indexes.size() == decoding_block_indexes.size(), "migrate_blocks: ",
                context_block_indexes.size(), " context blocks but ", decoding_block_indexes.size(),
                " decoding blocks");
    TORCH_CHECK(decoding_pp_size > 0 && decoding_tp_size > 0, "decoding parallel sizes must be positive");
    KvmGeom g;
    // the pool is the decoding rank's share: [blocks, L/dec_pp, H/dec_tp, B, D]
    g.num_layers = k_cache.size(1) * decoding_pp_size;
    g.num_kv_heads = k_cache.size(2) * decoding_tp_size;
    g.block_size = k_cache.size(3);
    g.head_dim = k_cache.size(4);
    g.dtype_bytes = (int64_t)k_cache.element_size();
    g.ctx_pp_size = (int32_t)context_pp_size;
    g.ctx_tp_size = (int32_t)context_tp_size;
    g.dec_pp_size = (int32_t)decoding_pp_size;
    g.dec_tp_size = (int32_t)decoding_tp_size;
    g.dec_pp_rank = (int32_t)decoding_pp_rank;
    g.dec_tp_rank = (int32_t)decoding_tp_rank;
    g.ctx_instance = context_instance;
    check(kvm_migrate(&g, context_block_indexes.data(), decoding_block_indexes.data(),
                      (int64_t)context_block_indexes.size(), k_cache.data_ptr(), v_cache.data_ptr(),
                      k_cache.size(0), current_stream(k_cache)),
          "migrate_blocks");
}

void migrate_blocks(int64_t context_pp_size, int64_t context_tp_size,
                    std::vector<int64_t> context_block_indexes, int64_t decoding_pp_size,
                    int64_t decoding_tp_size, int64_t decoding_pp_rank, int64_t decoding_tp_rank,
                    std::vector<int64_t> decoding_block_indexes, const at::Tensor &k_cache,
                    const at::Tensor &v_cache)
{
    migrate_blocks_from(0, context_pp_size, context_tp_size, std::move(context_block_indexes), decoding_pp_size,
                        decoding_tp_size, decoding_pp_rank, decoding_tp_rank, std::move(decoding_block_indexes),
                        k_cache, v_cache);
}

void swap(std::vector<int64_t> source_block_ids, std::vector<int64_t> target_block_ids, bool is_swap_in,
          const at::Tensor &k_cache, const at::Tensor &v_cache, const at::Tensor &k_swap,
          const at::Tensor &v_swap)
{
    check_pool(k_cache, "k_cache", true);
    check_pool(v_cache, "v_cache", true);
    check_pool(k_swap, "k_swap", false);
    check_pool(v_swap, "v_swap", false);
    TORCH_CHECK(k_cache.sizes() == v_cache.sizes() && k_swap.sizes() == v_swap.sizes(),
                "K and V pools must agree in shape");
    TORCH_CHECK(k_cache.sizes().slice(1) == k_swap.sizes().slice(1), "GPU and host pools must agree in block shape");
    TORCH_CHECK(k_cache.dtype() == v_cache.dtype() && k_cache.dtype() == k_swap.dtype() &&
                    k_cache.dtype() == v_swap.dtype(),
                "all four pools must share one dtype");
    TORCH_CHECK(source_block_ids.size() == target_block_ids.size(), "swap: ", source_block_ids.size(),
                " source blocks but ", target_block_ids.size(), " target blocks");
    const int64_t slab = k_cache.size(0) ? (int64_t)(k_cache.nbytes() / k_cache.size(0)) : 0;
    check(kvm_swap(source_block_ids.data(), target_block_ids.data(), (int64_t)source_block_ids.size(),
                   is_swap_in ? 1 : 0, k_cache.data_ptr(), v_cache.data_ptr(), k_swap.data_ptr(),
                   v_swap.data_ptr(), slab, k_cache.size(0), k_swap.size(0), current_stream(k_cache)),
          "swap");
}

}  // namespace

// The op namespaces are DistServe's.  A process that must also keep another library's
// registration of the same names (two definitions of one op are an error in torch) loads
// the build of this file with -DKVM_MIGRATION_NS=... -DKVM_SWAP_NS=... instead, and calls
// the ops under those names.
#ifndef KVM_MIGRATION_NS
#define KVM_MIGRATION_NS block_migration_ops
#endif
#ifndef KVM_SWAP_NS
#define KVM_SWAP_NS swapping_ops
#endif
#define KVM_TORCH_LIBRARY(ns, m) TORCH_LIBRARY(ns, m)

KVM_TORCH_LIBRARY(KVM_MIGRATION_NS, m)
{
    // structs, handles and signatures are only what this file was compiled against within one major version
    TORCH_CHECK(kvm_version() / 10000 == KVM_ABI_MAJOR, "libkvmove.so is version ", kvm_version(),
                ", this op library was built for major version ", KVM_ABI_MAJOR);
    m.def("get_ipc_mem_handle(Tensor t) -> int[]", get_ipc_mem_handle);
    m.def("register_ipc_mem_handle(int[] k_handle, int[] v_handle, int num_layers, int num_heads, "
          "int[] context_parallel_config, int[] decoding_parallel_config) -> ()",
          register_ipc_mem_handle);
    m.def("migrate_blocks(int context_pp_size, int context_tp_size, int[] context_block_indexes, "
          "int decoding_pp_size, int decoding_tp_size, int decoding_pp_rank, int decoding_tp_rank, "
          "int[] decoding_block_indexes, Tensor k_cache, Tensor v_cache) -> ()",
          migrate_blocks);
    m.def("register_ipc_mem_handle_from(int context_instance, int[] k_handle, int[] v_handle, int num_layers, "
          "int num_heads, int[] context_parallel_config, int[] decoding_parallel_config) -> ()",
          register_ipc_mem_handle_from);
    m.def("migrate_blocks_from(int context_instance, int context_pp_size, int context_tp_size, "
          "int[] context_block_indexes, int decoding_pp_size, int decoding_tp_size, int decoding_pp_rank, "
          "int decoding_tp_rank, int[] decoding_block_indexes, Tensor k_cache, Tensor v_cache) -> ()",
          migrate_blocks_from);
}

KVM_TORCH_LIBRARY(KVM_SWAP_NS, m)
{
    m.def("swap(int[] source_block_ids, int[] target_block_ids, bool is_swap_in, Tensor k_cache, "
          "Tensor v_cache, Tensor k_swap, Tensor v_swap) -> ()",
          swap);
}
