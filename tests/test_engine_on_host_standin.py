"""The engine's host logic without a GPU: a selection of the GPU parity tests (every pause path and option,
the state-machine edges beside the oracle, roll-back of a pause that cannot park its bytes, stale
registrations, the offload-free tag, seeded random process lives beside the oracle, the allocation-free
scan) run in a child pytest against the test-only build of the library's own sources on a host stand-in
of the HIP calls (tests/host_standin). What this holds is the part of the engine that is not a kernel:
planning, descriptor lists, batching, the copy / unmap / release threads, bookkeeping, error paths. The
kernels themselves, and everything timing-related, are only ever tested on the GPU (-m gpu)."""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "host_standin"))

SELECTION = ("option_paths or state_machine_edges or rolls_back or stale_registration or releases_without_copy or "
             "all_zero_and_tiny or mixed_callers or random_sequences_with_cycles_match_oracle or pool_reserved or "
             "paused_gate or without_allocation_equals or failed_allocation or known_answers or ragged")


def test_engine_logic_tests_pass_on_the_host_standin():
    import build_standin
    lib = build_standin.build(os.path.join(HERE, "host_standin", "_build"))
    env = dict(os.environ, AMEM_TEST_LIB=lib, AMEM_ENABLE="1", GMM_LOG="1")
    r = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "-p", "no:cacheprovider", "-k", SELECTION,
                        os.path.join(HERE, "test_gpu_cycle.py"), os.path.join(HERE, "test_gpu_kernels.py"),
                        os.path.join(HERE, "test_zz_no_alloc.py")],
                       env=env, capture_output=True, text=True, timeout=900, cwd=os.path.dirname(HERE))
    tail = (r.stdout + r.stderr)[-4000:]
    assert r.returncode == 0, tail
    m = re.search(r"(\d+) passed", r.stdout)
    assert m and int(m.group(1)) >= 20, tail
    assert "failed" not in r.stdout.splitlines()[-1], tail
