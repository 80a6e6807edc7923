"""ctypes binding of the kvmove C ABI (``include/kvmove.h``), one Python function per entry point.

Pointers are plain integers (``tensor.data_ptr()``), streams are ``hipStream_t`` values as
integers (``torch.cuda.current_stream().cuda_stream``).  A nonzero return code raises
``KvmError`` carrying ``kvm_last_error()``.

The module-level functions bind the package's own ``lib/libkvmove.so``.  ``Binding(path)``
binds any other build of the same interface with the same functions as methods (the tests
bind the exploration build, which has its own registry and options, beside the product).
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Sequence

KVM_OK = 0
KVM_EINVAL = -1
KVM_ERANGE = -2
KVM_EDUP = -3
KVM_ENOTREG = -4
KVM_EHIP = -5
KVM_EHANDLE = -6
KVM_EMISMATCH = -7
KVM_HANDLE_WORDS = 18
KVM_ABI_MAJOR = 1
KVM_IPC_MAX_ALLOC_BYTES = 1 << 31

# every symbol include/kvmove.h declares
EXPORTS = (
    "kvm_version", "kvm_last_error", "kvm_get_mem_handle", "kvm_register_mem_handle",
    "kvm_register_source", "kvm_reset", "kvm_opened_handles", "kvm_migrate", "kvm_swap", "kvm_copy_plain",
    "kvm_set_option", "kvm_get_option", "kvm_migrate_plan", "kvm_swap_plan", "kvm_debug_divide",
)


class KvmError(RuntimeError):
    def __init__(self, code: int, text: str):
        super().__init__(f"{text} (kvmove error {code})")
        self.code = code


class KvmGeom(ctypes.Structure):
    _fields_ = [
        ("num_layers", ctypes.c_int64), ("num_kv_heads", ctypes.c_int64), ("block_size", ctypes.c_int64),
        ("head_dim", ctypes.c_int64), ("dtype_bytes", ctypes.c_int64),
        ("ctx_pp_size", ctypes.c_int32), ("ctx_tp_size", ctypes.c_int32),
        ("dec_pp_size", ctypes.c_int32), ("dec_tp_size", ctypes.c_int32),
        ("dec_pp_rank", ctypes.c_int32), ("dec_tp_rank", ctypes.c_int32),
        ("ctx_instance", ctypes.c_int64),
    ]


def _lib_path() -> str:
    lib_dir = os.environ.get("KVMOVE_LIB_DIR") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
    return os.path.join(lib_dir, "libkvmove.so")


def _load(path: str) -> ctypes.CDLL:
    if not os.path.exists(path):
        raise RuntimeError(f"{os.path.basename(path)} not found at {path}; build it with "
                           "`python distserve_amd/csrc/build.py`")
    lib = ctypes.CDLL(path)
    i64, i32, vp, ip = ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64)
    lib.kvm_version.restype = ctypes.c_int
    lib.kvm_last_error.restype = ctypes.c_char_p
    # the shapes bound below are those of one major version; any other must not be called
    if lib.kvm_version() // 10000 != KVM_ABI_MAJOR:
        raise RuntimeError(f"{path} is kvmove version {lib.kvm_version()}; this binding is written for major "
                           f"version {KVM_ABI_MAJOR}")
    lib.kvm_get_mem_handle.argtypes = [vp, i64, ip]
    lib.kvm_register_mem_handle.argtypes = [ip, ip, i64, i64, ip, ip, i64]
    lib.kvm_register_source.argtypes = [i32, i32, i32, i32, i64, i64, vp, vp, i64, i64]
    lib.kvm_reset.argtypes = []
    lib.kvm_opened_handles.argtypes = []
    lib.kvm_opened_handles.restype = i64
    lib.kvm_migrate.argtypes = [ctypes.POINTER(KvmGeom), ip, ip, i64, vp, vp, i64, vp]
    lib.kvm_swap.argtypes = [ip, ip, i64, ctypes.c_int, vp, vp, vp, vp, i64, i64, i64, vp]
    lib.kvm_copy_plain.argtypes = [vp, vp, i64, vp]
    lib.kvm_set_option.argtypes = [ctypes.c_char_p, i64]
    lib.kvm_get_option.argtypes = [ctypes.c_char_p]
    lib.kvm_get_option.restype = i64
    lib.kvm_migrate_plan.argtypes = [ctypes.POINTER(KvmGeom), i64, vp, vp, i64, ip]
    lib.kvm_swap_plan.argtypes = [ip, ip, i64, i64, ctypes.c_int, i64, i64, ip]
    lib.kvm_debug_divide.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
    lib.kvm_debug_divide.restype = ctypes.c_uint32
    for name in EXPORTS:
        fn = getattr(lib, name)
        if name not in ("kvm_last_error", "kvm_get_option", "kvm_version", "kvm_debug_divide",
                        "kvm_opened_handles"):
            fn.restype = ctypes.c_int
    return lib


def _arr(values: Sequence[int]):
    if isinstance(values, ctypes.Array):
        return values
    return (ctypes.c_int64 * len(values))(*values)


def index_array(values: Sequence[int]):
    """A block-index list converted once, for callers that reuse it across calls."""
    return _arr(list(values))


def geom(num_layers, num_kv_heads, block_size, head_dim, dtype_bytes, ctx_pp=1, ctx_tp=1,
         dec_pp=1, dec_tp=1, dec_pp_rank=0, dec_tp_rank=0, ctx_instance=0) -> KvmGeom:
    return KvmGeom(num_layers, num_kv_heads, block_size, head_dim, dtype_bytes,
                   ctx_pp, ctx_tp, dec_pp, dec_tp, dec_pp_rank, dec_tp_rank, ctx_instance)


class Binding:
    """One loaded build of the library.  Every build has its own registry of context pools
    and its own options."""

    # names a caller may want beside the functions, so that a Binding can stand in for this module
    KvmError, KvmGeom = KvmError, KvmGeom
    KVM_OK, KVM_EINVAL, KVM_ERANGE, KVM_EDUP, KVM_ENOTREG = KVM_OK, KVM_EINVAL, KVM_ERANGE, KVM_EDUP, KVM_ENOTREG
    KVM_EHIP, KVM_EHANDLE, KVM_EMISMATCH = KVM_EHIP, KVM_EHANDLE, KVM_EMISMATCH
    KVM_HANDLE_WORDS, KVM_IPC_MAX_ALLOC_BYTES, EXPORTS = KVM_HANDLE_WORDS, KVM_IPC_MAX_ALLOC_BYTES, EXPORTS
    geom, index_array = staticmethod(geom), staticmethod(index_array)

    def __init__(self, path: str):
        self.path = path
        self.lib = _load(path)

    def _check(self, rc: int) -> None:
        if rc != KVM_OK:
            raise KvmError(rc, self.lib.kvm_last_error().decode())

    def version(self) -> int:
        return self.lib.kvm_version()

    def get_mem_handle(self, dev_ptr: int, nbytes: int) -> List[int]:
        out = (ctypes.c_int64 * KVM_HANDLE_WORDS)()
        self._check(self.lib.kvm_get_mem_handle(dev_ptr, nbytes, out))
        return list(out)

    def register_mem_handle(self, k_handle, v_handle, num_layers, num_kv_heads, context_pc, decoding_pc,
                            ctx_instance: int = 0) -> None:
        if len(k_handle) != KVM_HANDLE_WORDS or len(v_handle) != KVM_HANDLE_WORDS:
            raise KvmError(KVM_EHANDLE, f"a memory handle has {KVM_HANDLE_WORDS} words")
        if len(context_pc) != 4 or len(decoding_pc) != 4:
            raise KvmError(KVM_EINVAL, "parallel configs are [tp_size, tp_rank, pp_size, pp_rank]")
        self._check(self.lib.kvm_register_mem_handle(_arr(k_handle), _arr(v_handle), num_layers, num_kv_heads,
                                                     _arr(context_pc), _arr(decoding_pc), ctx_instance))

    def register_source(self, ctx_pp_size, ctx_tp_size, pp_rank, tp_rank, num_layers, num_kv_heads,
                        k_ptr: int, v_ptr: int, nbytes_each: int, ctx_instance: int = 0) -> None:
        self._check(self.lib.kvm_register_source(ctx_pp_size, ctx_tp_size, pp_rank, tp_rank, num_layers,
                                                 num_kv_heads, k_ptr, v_ptr, nbytes_each, ctx_instance))

    def reset(self) -> None:
        self._check(self.lib.kvm_reset())

    def opened_handles(self) -> int:
        """Allocations of other processes that registration currently keeps mapped."""
        return self.lib.kvm_opened_handles()

    def migrate(self, g: KvmGeom, ctx_idx: Sequence[int], dec_idx: Sequence[int], dst_k: int, dst_v: int,
                dst_num_blocks: int, stream: int = 0, n: int | None = None) -> None:
        n = len(ctx_idx) if n is None else n
        if n == len(ctx_idx) and len(ctx_idx) != len(dec_idx):
            raise KvmError(KVM_EINVAL, f"{len(ctx_idx)} context blocks but {len(dec_idx)} decoding blocks")
        self._check(self.lib.kvm_migrate(ctypes.byref(g), _arr(ctx_idx), _arr(dec_idx), n, dst_k, dst_v,
                                         dst_num_blocks, stream))

    def swap(self, src_ids: Sequence[int], dst_ids: Sequence[int], is_swap_in: bool, k_gpu: int, v_gpu: int,
             k_host: int, v_host: int, slab_bytes: int, n_gpu_blocks: int, n_host_blocks: int,
             stream: int = 0) -> None:
        if len(src_ids) != len(dst_ids):
            raise KvmError(KVM_EINVAL, f"{len(src_ids)} source blocks but {len(dst_ids)} target blocks")
        self._check(self.lib.kvm_swap(_arr(src_ids), _arr(dst_ids), len(src_ids), 1 if is_swap_in else 0, k_gpu,
                                      v_gpu, k_host, v_host, slab_bytes, n_gpu_blocks, n_host_blocks, stream))

    def copy_plain(self, dst: int, src: int, nbytes: int, stream: int = 0) -> None:
        self._check(self.lib.kvm_copy_plain(dst, src, nbytes, stream))

    def set_option(self, name: str, value: int) -> None:
        self._check(self.lib.kvm_set_option(name.encode(), value))

    def get_option(self, name: str) -> int:
        v = self.lib.kvm_get_option(name.encode())
        if v == KVM_EINVAL and self.lib.kvm_last_error():
            raise KvmError(KVM_EINVAL, self.lib.kvm_last_error().decode())
        return v

    def swap_plan(self, src_ids: Sequence[int], dst_ids: Sequence[int], slab_bytes: int, is_swap_in: bool = False,
                  n_gpu_blocks: int = 0, n_host_blocks: int = 0) -> dict:
        if len(src_ids) != len(dst_ids):
            raise KvmError(KVM_EINVAL, f"{len(src_ids)} source blocks but {len(dst_ids)} target blocks")
        out = (ctypes.c_int64 * 4)()
        self._check(self.lib.kvm_swap_plan(_arr(src_ids), _arr(dst_ids), len(src_ids), slab_bytes,
                                           1 if is_swap_in else 0, n_gpu_blocks, n_host_blocks, out))
        return dict(zip(("mode", "copies_per_pool", "launches", "workgroups_per_pool_kind"), list(out)))

    def migrate_plan(self, g: KvmGeom, n: int, dst_k: int, dst_v: int, dst_num_blocks: int = 0) -> dict:
        out = (ctypes.c_int64 * 10)()
        self._check(self.lib.kvm_migrate_plan(ctypes.byref(g), n, dst_k, dst_v, dst_num_blocks, out))
        keys = ("workgroups_per_block", "threads", "vector_bytes", "segments", "launches",
                "payload_bytes_per_block", "simple_kernel", "max_work_items", "vectors_per_lane",
                "pairs_per_launch")
        return dict(zip(keys, list(out)))

    def debug_divide(self, n: int, d: int) -> int:
        return self.lib.kvm_debug_divide(n, d)


default = Binding(_lib_path())
lib = default.lib

version = default.version
get_mem_handle = default.get_mem_handle
register_mem_handle = default.register_mem_handle
register_source = default.register_source
reset = default.reset
opened_handles = default.opened_handles
migrate = default.migrate
swap = default.swap
copy_plain = default.copy_plain
set_option = default.set_option
get_option = default.get_option
swap_plan = default.swap_plan
migrate_plan = default.migrate_plan
debug_divide = default.debug_divide
