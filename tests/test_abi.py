"""The C-ABI library loads without a GPU and exports exactly what
include/minuet_hip.h declares; the host-only entry points agree with the oracle."""
import ctypes
import os
import re

import numpy as np
import pytest

import minuet_oracle as orc
from minuet_amd.nn.functional import _C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "minuet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for match in re.finditer(r"\b(mnt_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = match.group(2).strip()
        count = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
        decls[match.group(1)] = count
    return decls


def test_library_exports_every_declared_symbol():
    lib = _C.load_library()
    decls = declared_functions()
    assert len(decls) >= 25
    for name in decls:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert lib.mnt_abi_version() == 1
    assert lib.mnt_last_error() == b""


def test_python_signatures_match_header():
    decls = declared_functions()
    assert set(decls) == set(_C.SIGNATURES), set(decls) ^ set(_C.SIGNATURES)
    for name, count in decls.items():
        assert len(_C.SIGNATURES[name][1]) == count, name


def test_exported_symbols_are_all_declared():
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", _C.library_path()], capture_output=True,
                         text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    exported = {s for s in exported if s.startswith("mnt_")}
    assert exported == set(declared_functions())


def test_no_oracle_or_cpu_fallback_in_product():
    """The product never imports the oracle and has no eager fallback."""
    for base, _, files in os.walk(os.path.join(ROOT, "minuet_amd")):
        for name in files:
            if name.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, name)).read()
                assert "minuet_oracle" not in text and "c_oracle" not in text, name
    import torch
    from minuet_amd.nn import functional as F
    cpu = torch.zeros((4, 3), dtype=torch.int32)
    for call in (lambda: F.arg_sort_coordinates(cpu), lambda: F.unique_coordinates(cpu),
                 lambda: F.query_sorted_index_with_offsets(cpu, cpu, cpu),
                 lambda: F.compute_kernel_map_sizes(cpu),
                 lambda: F.compute_kernel_map_masks(4, cpu, cpu),
                 lambda: F.sparse_convolution_forward(torch.zeros(4, 2), torch.zeros(1, 2, 2), cpu, cpu,
                                                      None, cpu, 1, 1)):
        with pytest.raises(NotImplementedError):
            call()


@pytest.mark.parametrize("threshold", [-1, 0.0, 0.15, 0.5, 2.0, None])
def test_padding_plan_matches_oracle(threshold):
    rng = np.random.default_rng(3)
    cases = [[1, 1, 1, 10], [0, 0, 0], [0, 0, 7], [5], [], [0, 0, 5, 6]]
    cases += [np.sort(rng.integers(0, 1000, size=rng.integers(1, 130))).tolist() for _ in range(40)]
    for sizes in cases:
        buckets = _C.generate_padding_buckets(sizes, threshold)
        assert buckets == orc.generate_padding_buckets(sizes, threshold)
        assert _C.cumsum_kernel_padded_sizes(sizes, buckets) == orc.cumsum_kernel_padded_sizes(sizes, buckets)


def test_padding_plan_rejects_bad_boundaries():
    with pytest.raises(RuntimeError, match=r"\[Minuet\].*bucket boundaries"):
        _C.cumsum_kernel_padded_sizes([1, 2, 3], [0, 2])
    assert _C.load_library().mnt_last_error().startswith(b"[Minuet]")
    _C.cuda_reset_error()
    assert _C.load_library().mnt_last_error() == b""


def test_one_caller_thread_per_stream():
    """A second thread that enters the library on a stream another thread holds
    fails with a message instead of racing; after the release it gets through."""
    import threading
    lib = _C.load_library()
    results = {}

    def other(tag):
        status = lib.mnt_buffer_set_growth(None, ctypes.c_float(1.0))
        results[tag] = (status, lib.mnt_last_error().decode())

    _C.stream_acquire(None)
    try:
        assert lib.mnt_buffer_set_growth(None, ctypes.c_float(1.0)) == 0      # the holder itself gets through
        worker = threading.Thread(target=other, args=("held",))
        worker.start()
        worker.join()
    finally:
        _C.stream_release(None)
    worker = threading.Thread(target=other, args=("free",))
    worker.start()
    worker.join()
    status, message = results["held"]
    assert status != 0 and "in use by another thread" in message and message.startswith("[Minuet]")
    assert results["free"][0] == 0
    # a stream nobody holds is unaffected by the hold on another one
    _C.stream_acquire(None)
    try:
        side = ctypes.c_void_p(0x1000)          # never dereferenced: only names the registry entry
        done = {}

        def elsewhere():
            done["status"] = lib.mnt_buffer_set_growth(side, ctypes.c_float(1.0))
        worker = threading.Thread(target=elsewhere)
        worker.start()
        worker.join()
        assert done["status"] == 0
    finally:
        _C.stream_release(None)
