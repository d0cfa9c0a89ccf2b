"""The host bookkeeping of the cache (block pool with page ids in one arena, sequence table, step
arrays written in place) under AddressSanitizer and UndefinedBehaviorSanitizer: a native driver
(tests/native/fuzz_bookkeeping.cc) runs seeded random operation sequences -- add / remove / fork /
popn / sliding windows / prefill, decode and token-tree steps with commits / clear, invalid ones
included -- and checks after every step that page ids and append slots stay inside the pool, that no
slot is handed out twice and that nothing is written behind the step buffer.  Host code only: the
sanitizers never see a GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROCM_INCLUDE = "/opt/rocm/include"


@pytest.fixture(scope="module")
def fuzz_binary(tmp_path_factory):
    gxx = shutil.which("g++")
    if gxx is None or not os.path.isdir(ROCM_INCLUDE):
        pytest.skip("needs g++ and the HIP headers")
    exe = str(tmp_path_factory.mktemp("fuzz") / "fuzz_bookkeeping")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-D__HIP_PLATFORM_AMD__", "-I" + ROCM_INCLUDE,
           os.path.join(ROOT, "tests", "native", "fuzz_bookkeeping.cc"),
           os.path.join(ROOT, "tvm_amd", "csrc", "kv_bookkeeping.cc"), "-o", exe]
    built = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert built.returncode == 0, built.stderr[-4000:]
    return exe


@pytest.mark.parametrize("sliding", [0, 1])
@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_random_operation_sequences_under_sanitizers(fuzz_binary, seed, sliding):
    # the harness of this environment preloads a library of its own; the sanitizer runtime only insists on coming first
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([fuzz_binary, str(seed), "3000", str(sliding)], capture_output=True, text=True, timeout=300,
                         env=env)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert "operations" in run.stdout


def test_window_that_cannot_slide_is_an_error_not_a_crash():
    """A shared prefix longer than the window: the reference erases pages past the end of the last block's
    page list (paged_kv_cache.cc:1966-1972); the library and the oracle refuse the step."""
    from oracle.host_cache import CacheError, HostCache
    from tvm_amd import KVError
    from tvm_amd import get_global_func as gf

    def drive(cache, add, fork, enable, begin):
        add(0)
        begin([0], [40])
        fork(0, 1, 40)
        enable(1, 8, 0)
        begin([1], [3])

    oracle = HostCache([4, 512, 64, 16, 1], rope_mode=2)
    with pytest.raises(CacheError, match="sliding window has to drop"):
        drive(oracle, oracle.add_sequence, oracle.fork_sequence, oracle.enable_sliding_window_for_seq,
              lambda ids, lens: oracle.begin_forward(ids, lens))
    cache = gf("vm.builtin.paged_attention_kv_cache_create")([4, 512, 64, 16, 1], [0, 1], 8, 2, 64, 64, [0], False, 2,
                                                             1.0, 1e4, None, None)
    with pytest.raises(KVError, match="sliding window has to drop"):
        drive(cache, lambda s: gf("vm.builtin.kv_state_add_sequence")(cache, s),
              lambda p, c, pos: gf("vm.builtin.kv_state_fork_sequence")(cache, p, c, pos),
              lambda s, w, k: gf("vm.builtin.attention_kv_cache_enable_sliding_window_for_seq")(cache, s, w, k),
              lambda ids, lens: gf("vm.builtin.kv_state_begin_forward")(cache, ids, lens, None))
