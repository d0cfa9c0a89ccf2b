"""MI355X-native paged KV-cache attention behind the interface of apache/tvm's
``PagedAttentionKVCache``.

The product is ``lib/libtvmkv.so`` (C ABI, ``include/tvmkv.h``): hand-written gfx950 HIP
kernels plus the host-side page pool.  This package is the Python face of it, shaped like the
reference's own Python entry points: ``get_global_func("vm.builtin.kv_state_add_sequence")``
and friends return callables with the reference's argument order
(src/runtime/vm/kv_state.cc:33-116 of the reference), and ``tvm_amd.kernels`` exposes the
kernel launchers with the argument order of the reference's kernel slots.
"""
from ._lib import LIB_PATH, KVError, decode_split_plan, lib, set_option  # noqa: F401
from .runtime import AttnKind, RopeMode, Shape, get_global_func  # noqa: F401
