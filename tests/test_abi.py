"""The C-ABI library loads and exports every symbol the public header declares."""
import ctypes
import os
import re
import shutil
import subprocess

import pytest

from aptserve_hip import _lib, probes

LIBS = [(_lib.LIB_PATH, _lib.HEADER), (probes.LIB_PATH, probes.HEADER)]


@pytest.mark.parametrize("lib_path,header", LIBS, ids=["product", "probes"])
def test_header_parses_and_every_symbol_is_exported(lib_path, header):
    protos = _lib.parse_header(header)
    if header == _lib.HEADER:
        assert "aps_hidden_to_cache" in protos and "aps_cache_to_hidden" in protos
        assert "aps_mixed_kv_to_cache" in protos and "aps_decode_step_cache_ops" in protos
    lib = ctypes.CDLL(str(lib_path))
    for name in protos:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"


@pytest.mark.parametrize("lib_path,header", LIBS, ids=["product", "probes"])
def test_no_undeclared_exports(lib_path, header):
    out = subprocess.run(["nm", "-D", "--defined-only", str(lib_path)], capture_output=True, text=True).stdout
    exported = set(re.findall(r" T (aps_\w+)", out))
    assert exported == set(_lib.parse_header(header)), "header and library disagree about the ABI"


def test_product_abi_holds_no_measurement_kernels():
    """The library a maintainer of the reference binds exports operators only: the copy / stream / matrix-core
    probes of the benchmark live in a library of their own."""
    protos = set(_lib.parse_header())
    assert not {n for n in protos if "probe" in n or n == "aps_copy_bytes"}
    assert {"aps_copy_bytes", "aps_stream_probe", "aps_mfma_probe"} == set(_lib.parse_header(probes.HEADER))


def test_loader_sets_prototypes_and_version():
    lib = _lib.load()
    assert lib.aps_abi_version() == _lib._abi_version_of_header()
    assert lib.aps_status_string(0) == b"ok"
    assert lib.aps_status_string(-1) == b"invalid argument"


def test_signatures_carry_no_torch_types():
    text = _lib.HEADER.read_text()
    assert "torch" not in text.lower().replace("pytorch", "")
    assert "at::" not in text and "Tensor" not in text


def test_argument_errors_return_without_launching():
    lib = _lib.load()
    # negative sizes / null pointers are rejected on the host, before any GPU call
    pl = probes.load()
    assert pl.aps_copy_bytes(None, None, -1, None) == -1
    assert pl.aps_copy_bytes(None, None, 0, None) == 0
    assert lib.aps_hidden_to_cache(None, None, None, None, None, 0, 768, 768, 768, 0, 0, 0, 2, None) == 0
    assert lib.aps_hidden_to_cache(None, None, None, None, None, 4, 768, 768, 768, 0, 0, 0, 2, None) == -1
    assert lib.aps_hidden_to_cache(None, None, None, None, None, 4, 768, 768, 768, 0, 0, 0, 3, None) == -1
    # prompt attention: a zero, negative or non-finite softmax scale is rejected on the host
    for bad in (0.0, -1.0, float("nan"), float("inf")):
        assert lib.aps_varlen_prefill_attention(16, 16, 16, 16, 16, 1, 8, 8, 2, 64, 128, 128, 128, 128, bad, 0, None) == -1
    # the matrix-core probe: unknown shape / dtype / null buffers are errors, an empty launch is not
    assert pl.aps_mfma_probe(7, 0, 16, 16, 1, 1, None) == -1
    assert pl.aps_mfma_probe(-1, 0, 16, 16, 1, 1, None) == -1
    assert pl.aps_mfma_probe(0, 5, 16, 16, 1, 1, None) == -1
    assert pl.aps_mfma_probe(0, 0, None, None, 1, 1, None) == -1
    assert pl.aps_mfma_probe(1, 0, 16, 16, 0, 1, None) == 0


def test_jobs_are_planned_on_the_host_and_checked_before_a_launch():
    """Planning a job is arithmetic on the arguments (no GPU call, so made-up addresses will do here): the checks of
    the direct call, a buffer of the promised size, and launches that refuse what no planning call wrote.  A job
    over an empty batch launches nothing and is not an error, also through the hybrid call."""
    import ctypes
    lib = _lib.load()
    A = 1 << 20                                           # an aligned address that is never dereferenced
    H, D, BS, B, W = 40, 128, 16, 4, 8
    job = (ctypes.c_uint64 * 40)()
    ja = ctypes.addressof(job)
    assert ctypes.sizeof(job) == 320                      # APS_ATTENTION_JOB_BYTES = APS_CACHE_JOB_BYTES

    def plan_attention(addr, nbytes, batch, q_dtype=0, head_size=D):
        return lib.aps_paged_decode_attention_job(addr, nbytes, A, A, A, A, None, None, A, None, A, batch, H, head_size,
                                                  BS, W, W, 0, H * head_size, H * head_size, BS * H * head_size, 64, 0,
                                                  0, W * BS, 0, 0.1, q_dtype, q_dtype, 1.0, 1.0, None, 0)

    assert plan_attention(ja, 320, B) == 0
    assert plan_attention(ja, 64, B) == -1                # buffer too small
    assert plan_attention(ja + 4, 320, B) == -1           # not 8-byte aligned
    assert plan_attention(None, 320, B) == -1
    assert plan_attention(ja, 320, -1) == -1              # the direct call's checks
    assert plan_attention(ja, 320, B, q_dtype=7) == -2    # unsupported dtype
    assert plan_attention(ja, 320, B, head_size=48) == -2
    junk = (ctypes.c_uint64 * 40)()
    assert lib.aps_attention_job_launch(ctypes.addressof(junk), None) == -1
    assert lib.aps_cache_job_launch(ctypes.addressof(junk), None) == -1
    assert lib.aps_attention_job_launch(None, None) == -1 and lib.aps_cache_job_launch(None, None) == -1
    # empty jobs: planned, launched (nothing to do), and accepted by the hybrid call without sequences
    assert plan_attention(ja, 320, 0) == 0 and lib.aps_attention_job_launch(ja, None) == 0
    store = (ctypes.c_uint64 * 40)()
    sa = ctypes.addressof(store)
    plan_store = lambda n_store, n_kv, elem=2: lib.aps_decode_step_cache_ops_job(
        sa, 320, None, A, A, None, 0, A, A, A, n_store, B, H * D, 0, H * D, H * D, 64 * BS, A, A, A, A, A, A, n_kv,
        H * D, H * D, BS, BS * H * D, 64, elem)
    assert plan_store(0, 0) == 0 and lib.aps_cache_job_launch(sa, None) == 0
    assert plan_store(2, -1) == -1 and plan_store(2, 2, elem=3) == -1
    assert plan_store(0, 0) == 0
    assert lib.aps_hybrid_decode_attention(sa, ja, None, 0, None, 0, None, 0, 0, None, None, 0, 0, None, None, None, 0,
                                           H, D, 0.1, None, 0, 0, 0, None, 0, None) == 0
    assert lib.aps_hybrid_decode_attention(ctypes.addressof(junk), None, None, 0, None, 0, None, 0, 0, None, None, 0, 0,
                                           None, None, None, 0, H, D, 0.1, None, 0, 0, 0, None, 0, None) == -1


def test_linear_workspace_planning_is_host_only_and_consistent():
    """aps_linear_nt_splits / _workspace_bytes are pure host functions (no launch): the workspace is the fp32
    partial tiles of every split, few-row products are split into whole 512-element chunks of K, and no plan asks
    for more workgroups than the part has CUs unless the output tiles alone already do."""
    lib = _lib.load()
    shapes = [(5120, 5120), (10240, 5120), (15360, 5120), (20480, 5120), (5120, 20480), (256, 64), (1536, 768)]
    for n, k in shapes:
        for m in (1, 2, 3, 5, 16, 17, 48, 49, 64, 128, 129, 192, 256, 300, 700, 1024, 4096, 16384):
            s = lib.aps_linear_nt_splits(m, n, k)
            assert s >= 1
            ws = lib.aps_linear_nt_workspace_bytes(m, n, k)
            if s > 1:
                assert ws == s * m * n * 4
            elif ws:
                # tail split of a large product: fp32 images of the parts of the tiles beyond the last full
                # round of 256 compute units; the parts fit one round
                tile_bytes = 256 * 256 * 4
                tiles = -(-m // 256) * (n // 256)
                rest = tiles % 256
                assert tiles > 256 and rest and ws % tile_bytes == 0
                ways = ws // tile_bytes // rest
                assert 2 <= ways <= 4 and ways * rest <= 256 and ws == ways * rest * tile_bytes
            if m <= 2:
                assert s == 1                                  # one launch of the dot-product kernel
            elif m <= 8 and k in (2048, 4096, 5120, 6144):
                assert s == 1 and ws == 0                      # K split inside the workgroups: nothing to add
            elif m <= 48:
                # whole 512-element chunks of K; workgroups of 64..128 weight rows, at most one per compute unit
                chunks = -(-k // 512)
                assert s <= chunks
                rows = 16 if m <= 16 else (32 if m <= 32 else 48)
                tiles = -(-n // 128) * -(-m // rows)
                assert s == 1 or tiles * s <= 256
            else:
                assert s == 1 or (n // 256) * s <= 256         # at least one row of tiles
    # degenerate arguments plan nothing
    assert lib.aps_linear_nt_splits(0, 5120, 5120) == 1 and lib.aps_linear_nt_workspace_bytes(0, 5120, 5120) == 0


def test_absorbed_attention_workspace_planning_is_host_only():
    """The workspace of the attention on hidden rows covers at least its named buffers (query image and context
    rows: n*H*Hd 16-bit each; fp32 scores over the padded longest sequence; a row of zeros), grows with the
    batch, and degenerate arguments plan nothing."""
    lib = _lib.load()
    f = lib.aps_absorbed_attention_workspace_bytes
    for heads, d in ((12, 64), (40, 128)):
        hd = heads * d
        prev = 0
        for n in (1, 2, 8, 16, 17, 128, 300, 5000):
            for max_len in (1, 33, 700, 2048):
                lp = -(-max_len // 32) * 32
                need = 2 * n * heads * hd * 2 + n * heads * lp * 4 + hd * 2
                got = f(n, max_len, heads, d)
                assert got >= need and got % 256 == 0, (n, max_len, heads, d, got, need)
            # small batches carry the partial sums of their token partitions as well: growth is only monotonic
            # once no sequence is split
            if n >= 300:
                assert f(n, 2048, heads, d) > prev
                prev = f(n, 2048, heads, d)
    assert f(0, 100, 40, 128) == 0 and f(4, 0, 40, 128) == 0


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs a C compiler")
def test_header_binds_from_plain_c(tmp_path):
    """A C99 program that includes the header, links the library and calls entry points that need no GPU: what
    a cgo / JNI / FFI binding of the reference's maintainers would do first."""
    src = tmp_path / "bind.c"
    src.write_text(r"""
#include <stdio.h>
#include <string.h>
#include "aptserve_hip.h"
int main(void) {
  if (aps_abi_version() != APS_ABI_VERSION) return 1;
  if (strcmp(aps_status_string(APS_OK), "ok") != 0) return 2;
  /* argument errors are reported as negative statuses before anything is launched */
  if (aps_hidden_to_cache(NULL, NULL, NULL, NULL, NULL, -1, 0, 0, 0, 0, 0, 0, 0, NULL) >= 0) return 3;
  if (aps_linear_nt_workspace_bytes(12, 5120, 5120) <= 0) return 4;     /* a dozen rows: K split over workgroups */
  if (aps_linear_nt_workspace_bytes(5, 5120, 5120) != 0) return 6;      /* a handful: split inside the workgroups */
  if (aps_decode_attention_workspace_bytes(4, 40, 128, 8192, 512) <= 0) return 5;   /* 16 partitions: flat path */
  printf("abi %d static scratch %d bytes\n", aps_abi_version(), (int)APS_STATIC_SCRATCH_BYTES);
  return 0;
}
""")
    exe = tmp_path / "bind"
    libdir = str(_lib.LIB_PATH.parent)
    rocm = "/opt/rocm/lib"
    cmd = ["gcc", "-std=c99", "-Wall", "-Werror", "-I", str(_lib.HEADER.parent), str(src), "-o", str(exe), "-L", libdir,
           "-l:" + _lib.LIB_PATH.name, "-Wl,-rpath," + libdir, "-Wl,-rpath," + rocm, "-Wl,-rpath-link," + rocm]
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr
    env = dict(os.environ, LD_LIBRARY_PATH=os.pathsep.join(filter(None, [rocm, os.environ.get("LD_LIBRARY_PATH")])))
    ran = subprocess.run([str(exe)], capture_output=True, text=True, env=env)
    assert ran.returncode == 0, (ran.returncode, ran.stdout, ran.stderr)
    assert ran.stdout.startswith("abi ")
