"""The C-ABI library loads, exports every symbol include/kvmove.h declares and refuses
malformed arguments without touching a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "kvmove.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kvm_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported(kvm):
    names = declared_symbols()
    assert len(names) >= 12 and set(names) == set(kvm.EXPORTS)
    raw = ctypes.CDLL(os.path.join(ROOT, "distserve_amd", "lib", "libkvmove.so"))
    for name in names:
        assert getattr(raw, name) is not None


def test_version_and_options(kvm, kvm_explore):
    header = open(os.path.join(ROOT, "include", "kvmove.h")).read()
    major = int(re.search(r"#define KVM_ABI_MAJOR (\d+)", header).group(1))
    words = int(re.search(r"#define KVM_HANDLE_WORDS (\d+)", header).group(1))
    assert kvm.version() // 10000 == major and kvm.KVM_HANDLE_WORDS == words
    assert kvm.get_option("xcd_map") == 1 and kvm.get_option("sort_pairs") == 1
    old = kvm.get_option("swap_wgs")
    kvm.set_option("swap_wgs", 12)
    assert kvm.get_option("swap_wgs") == 12
    kvm.set_option("swap_wgs", old)
    for name, bad in (("swap_mode", 4), ("swap_wgs", 0), ("swap_wgs_in", 5000), ("swap_kernel_below", -1),
                      ("xcd_map", 4), ("sort_pairs", 3), ("nope", 1)):
        with pytest.raises(kvm.KvmError) as e:
            kvm.set_option(name, bad)
        assert e.value.code == kvm.KVM_EINVAL
    # the product carries one kernel flavour and none of the knobs that select others ...
    for name in ("tile_bytes", "threads", "unroll", "nt_load", "nt_store", "wave_contig", "lds_pad", "simple"):
        with pytest.raises(kvm.KvmError):
            kvm.get_option(name)
        with pytest.raises(kvm.KvmError):
            kvm.set_option(name, 0)
    # ... the exploration build has them, with the product's flavour as the default
    x = kvm_explore
    assert x.version() == kvm.version()
    assert x.get_option("tile_bytes") == 0 and x.get_option("threads") == 64 and x.get_option("unroll") == 1
    assert x.get_option("nt_load") == 1 and x.get_option("nt_store") == 1 and x.get_option("simple") == 1
    x.set_option("unroll", 8)
    assert x.get_option("unroll") == 8
    x.set_option("unroll", 1)
    for name, bad in (("tile_bytes", 5000), ("threads", 100), ("unroll", 3), ("nt_store", 2), ("max_pairs", 865)):
        with pytest.raises(x.KvmError) as e:
            x.set_option(name, bad)
        assert e.value.code == x.KVM_EINVAL


def test_swap_plan_takes_the_kernel_by_default_and_the_engines_above_a_threshold(kvm):
    """Default: the copy kernel whatever the slab size, with its own workgroup count per
    direction.  With a "swap_kernel_below" threshold, calls whose copies average that many
    bytes go to the copy engines; runs of blocks consecutive on both sides count as one copy."""
    assert kvm.get_option("swap_mode") == 3 and kvm.get_option("swap_kernel_below") == 1 << 32
    assert kvm.get_option("swap_wgs") == 16 and kvm.get_option("swap_wgs_in") == 16
    scattered = ([5, 9, 2, 7], [1, 8, 3, 6])
    assert kvm.swap_plan(*scattered, 4 << 20) == {"mode": 1, "copies_per_pool": 4, "launches": 1,
                                                  "workgroups_per_pool_kind": 16}
    kvm.set_option("swap_wgs_in", 18)
    assert kvm.swap_plan(*scattered, 4 << 20, is_swap_in=True)["workgroups_per_pool_kind"] == 18
    kvm.set_option("swap_wgs_in", 16)
    # pools of unknown size: 432 blocks per launch; pools of at most 65536 blocks: 864
    ids = (list(range(0, 2000, 2)), list(range(1000)))
    assert kvm.swap_plan(*ids, 4096)["launches"] == 3
    assert kvm.swap_plan(*ids, 4096, n_gpu_blocks=4096, n_host_blocks=65536)["launches"] == 2
    assert kvm.swap_plan(*ids, 4096, n_gpu_blocks=4096, n_host_blocks=65537)["launches"] == 3
    assert kvm.swap_plan([], [], 4096) == {"mode": 2, "copies_per_pool": 0, "launches": 0, "workgroups_per_pool_kind": 0}
    kvm.set_option("swap_kernel_below", 2 << 20)
    try:
        assert kvm.swap_plan(*scattered, 4 << 20) == {"mode": 2, "copies_per_pool": 4, "launches": 0,
                                                      "workgroups_per_pool_kind": 0}
        assert kvm.swap_plan(*scattered, 2 << 20)["mode"] == 2
        assert kvm.swap_plan(*scattered, (2 << 20) - 16)["mode"] == 1
        # 8 consecutive blocks of 288 KiB are one 2.25 MiB copy; broken in two they are not
        run = list(range(10, 18))
        assert kvm.swap_plan(run, list(range(40, 48)), 288 << 10) == {"mode": 2, "copies_per_pool": 1, "launches": 0,
                                                                       "workgroups_per_pool_kind": 0}
        assert kvm.swap_plan(run, list(range(40, 44)) + list(range(50, 54)), 288 << 10)["mode"] == 1
        assert kvm.swap_plan(run, run[::-1], 288 << 10)["copies_per_pool"] == 8
        assert kvm.swap_plan(list(range(1000)), list(range(1000)), 4096)["mode"] == 2          # one 4 MiB run
        kvm.set_option("swap_kernel_below", 0)
        assert kvm.swap_plan(*scattered, 1024)["mode"] == 2
    finally:
        kvm.set_option("swap_kernel_below", 1 << 32)
    # forced modes are reported as they are
    for mode in (0, 1, 2):
        kvm.set_option("swap_mode", mode)
        assert kvm.swap_plan(*scattered, 4 << 20)["mode"] == mode
    kvm.set_option("swap_mode", 3)
    with pytest.raises(kvm.KvmError) as e:
        kvm.swap_plan([0], [0], 0)
    assert e.value.code == kvm.KVM_EINVAL
    with pytest.raises(kvm.KvmError) as e:
        kvm.swap_plan([-1], [0], 64)
    assert e.value.code == kvm.KVM_ERANGE


def test_argument_errors_need_no_gpu(kvm, fresh_registry):
    g = kvm.geom(4, 4, 16, 8, 2)
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate(g, [0], [0], 0, 0, 4)                       # null destination
    assert e.value.code == kvm.KVM_EINVAL
    bad = kvm.geom(5, 4, 16, 8, 2, ctx_pp=2)                    # 5 layers over pp 2
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate(bad, [0], [0], 4096, 8192, 4)
    assert e.value.code == kvm.KVM_EINVAL and "divisible" in str(e.value)
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate(kvm.geom(4, 4, 16, 8, 2, dec_tp=2, dec_tp_rank=2), [0], [0], 4096, 8192, 4)
    assert e.value.code == kvm.KVM_EINVAL
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate(g, [0], [0], 4096, 8192, 4)                 # nothing registered
    assert e.value.code == kvm.KVM_ENOTREG
    kvm.migrate(g, [], [], 4096, 8192, 4)                       # an empty list is a no-op even then
    with pytest.raises(kvm.KvmError) as e:
        kvm.register_mem_handle([0] * kvm.KVM_HANDLE_WORDS, [0] * kvm.KVM_HANDLE_WORDS, 4, 4, [1, 0, 1, 0], [1, 0, 1, 0])
    assert e.value.code == kvm.KVM_EHANDLE
    with pytest.raises(kvm.KvmError) as e:
        kvm.swap([0], [0], True, 0, 0, 0, 0, 64, 1, 1)
    assert e.value.code == kvm.KVM_EINVAL


def test_launches_stay_below_the_grid_limit_for_blocks_of_any_size(kvm, kvm_explore, fresh_registry):
    """A launch is 2 x tiles x blocks workgroups of `threads` lanes; the runtime refuses 2^32
    work-items and more, so the block list is split over more launches before anything is
    enqueued.  Pure arithmetic: null pools, nothing registered, no device."""
    plan = kvm.migrate_plan(kvm.geom(32, 32, 16, 128, 2), 909, 0, 0)          # LLaMA-2-7B, 1 -> 1, pools of any size
    assert plan["launches"] == 3 and plan["simple_kernel"] == 1 and plan["max_work_items"] == 2 * 4096 * 432 * 64
    assert plan["pairs_per_launch"] == 432 and plan["threads"] == 64 and plan["vectors_per_lane"] == 1
    plan = kvm.migrate_plan(kvm.geom(32, 32, 16, 128, 2), 909, 0, 0, 4096)    # ... pools of 4096 blocks: packed pairs
    assert plan["launches"] == 2 and plan["pairs_per_launch"] == 864 and plan["max_work_items"] == 2 * 4096 * 864 * 64
    assert kvm.migrate_plan(kvm.geom(32, 32, 16, 128, 2), 909, 0, 0, 65537)["pairs_per_launch"] == 432
    big = kvm.geom(128, 128, 256, 128, 2)                                      # 1 GiB per pool kind per block
    tiles = (1 << 30) // 1024
    for n in (1, 31, 32, 433, 5000):
        plan = kvm.migrate_plan(big, n, 0, 0, 4096)
        per_launch = (2**32 - 1) // (2 * 64) // tiles                          # 31, short of the padding allowance
        assert plan["payload_bytes_per_block"] == 2 << 30
        assert plan["launches"] == -(-n // per_launch)
        assert 0 < plan["max_work_items"] < 2**32
    for threads, unroll in ((256, 4), (1024, 4)):
        kvm_explore.set_option("threads", threads)
        kvm_explore.set_option("unroll", unroll)
        try:
            plan = kvm_explore.migrate_plan(big, 5000, 0, 0, 4096)
            assert plan["threads"] == threads and plan["vectors_per_lane"] == unroll
            assert 0 < plan["max_work_items"] < 2**32
        finally:
            kvm_explore.set_option("threads", 64)
            kvm_explore.set_option("unroll", 1)
    # with real (non-null) destination pointers the plan wants the sources registered, as before
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate_plan(big, 4, 4096, 8192)
    assert e.value.code == kvm.KVM_ENOTREG


def test_torch_ops_are_registered_with_the_reference_argument_order():
    import torch

    import distserve_amd  # noqa: F401  (loads the shim)

    s = str(torch.ops.block_migration_ops.migrate_blocks.default._schema)
    order = ["context_pp_size", "context_tp_size", "context_block_indexes", "decoding_pp_size", "decoding_tp_size",
             "decoding_pp_rank", "decoding_tp_rank", "decoding_block_indexes", "k_cache", "v_cache"]
    assert [s.index(a) for a in order] == sorted(s.index(a) for a in order)
    s = str(torch.ops.swapping_ops.swap.default._schema)
    order = ["source_block_ids", "target_block_ids", "is_swap_in", "k_cache", "v_cache", "k_swap", "v_swap"]
    assert [s.index(a) for a in order] == sorted(s.index(a) for a in order)
    s = str(torch.ops.block_migration_ops.register_ipc_mem_handle.default._schema)
    order = ["k_handle", "v_handle", "num_layers", "num_heads", "context_parallel_config", "decoding_parallel_config"]
    assert [s.index(a) for a in order] == sorted(s.index(a) for a in order)
    assert "int[]" in str(torch.ops.block_migration_ops.get_ipc_mem_handle.default._schema)
    # the forms that name a context instance are the same schemas behind one leading argument
    for name in ("register_ipc_mem_handle", "migrate_blocks"):
        plain = str(getattr(torch.ops.block_migration_ops, name).default._schema).split("(", 1)[1]
        named = str(getattr(torch.ops.block_migration_ops, name + "_from").default._schema).split("(", 1)[1]
        assert named == "int context_instance, " + plain
    # no CPU fallback: a CPU tensor is refused, loudly
    z = torch.zeros(2, 1, 1, 2, 2, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.block_migration_ops.migrate_blocks(1, 1, [0], 1, 1, 0, 0, [0], z, z)


def test_row_of_a_tile_is_computed_without_a_divider_exactly(kvm):
    """The kernel finds a tile's row as tile / pieces_per_row with a host-made multiplier and
    two shifts; the host twin of that arithmetic must equal plain division everywhere."""
    import random

    rng = random.Random(7)
    divisors = list(range(1, 70)) + [80, 96, 127, 128, 129, 255, 256, 257, 1000, 4095, 4096, 4097, 65535, 65536,
                                     65537, 2**20 - 1, 2**20, 2**20 + 1, 2**31 - 1, 2**31, 2**31 + 1, 2**32 - 1]
    divisors += [rng.randrange(1, 2**32) for _ in range(200)]
    for d in divisors:
        probes = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 3 * d + 1, 2**31 - 1, 2**31, 2**32 - 1, 2**32 - d]
        probes += [k * d + r for k in (5, 1023, 65535) for r in (0, d - 1)]
        probes += [rng.randrange(0, 2**32) for _ in range(40)]
        for n in probes:
            if 0 <= n < 2**32:
                assert kvm.debug_divide(n, d) == n // d, (n, d)
    assert kvm.debug_divide(5, 0) == 2**32 - 1


def test_the_package_refuses_to_import_without_its_libraries(tmp_path):
    """No CPU fallback: without the built HIP library the package fails at import, loudly."""
    import subprocess
    import sys

    env = dict(os.environ, KVMOVE_LIB_DIR=str(tmp_path))
    run = subprocess.run([sys.executable, "-c", "import distserve_amd"], capture_output=True, text=True, env=env,
                         cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert run.returncode != 0
    assert "libkvmove.so" in run.stderr and "build" in run.stderr.lower()


def test_the_alternate_namespace_build_registers_the_same_schemas_beside_the_first():
    """A process that keeps another library's block_migration_ops / swapping_ops loads the
    second build of the shim; both can live in one process."""
    import torch

    import distserve_amd

    torch.ops.load_library(os.path.join(os.path.dirname(distserve_amd.TORCH_LIB_PATH), "libkvmove_torch_alt.so"))

    def args_of(op):
        return str(op.default._schema).split("(", 1)[1]

    for name in ("get_ipc_mem_handle", "register_ipc_mem_handle", "migrate_blocks"):
        assert args_of(getattr(torch.ops.kvmove_block_migration_ops, name)) == \
            args_of(getattr(torch.ops.block_migration_ops, name))
    assert args_of(torch.ops.kvmove_swapping_ops.swap) == args_of(torch.ops.swapping_ops.swap)


def test_the_ceiling_probe_is_built_and_explains_its_flags():
    """The stand-alone probe of the memory system's ceilings (a fixture of the bench-target
    test) is built (no GPU call happens before its arguments are read)."""
    import subprocess

    probe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hbm_probe", "hbm_probe")
    assert os.path.exists(probe), "make -C tests/hbm_probe builds it"
    run = subprocess.run([probe, "--no-such-flag"], capture_output=True, text=True)
    assert run.returncode == 2
    assert "--section" in run.stderr and "--quick" in run.stderr
