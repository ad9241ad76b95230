"""Host-side logic that needs no GPU: synthetic inputs, the C-ABI library's
exports and its argument checks (which return before any launch), the Python
mirror's own checks."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from renee_amd import synth
from renee_amd._lib import EXPORTS, lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_positives_are_canonical_and_seeded():
    c = synth.CONFIGS[2]
    P = synth.make_positives(c["B"], 131072, c["kmax"], c["kmean"], c["zipf"], seed=3)
    Q = synth.make_positives(c["B"], 131072, c["kmax"], c["kmean"], c["zipf"], seed=3)
    assert np.array_equal(P.rowptr, Q.rowptr) and np.array_equal(P.colidx, Q.colidx)
    assert P.rowptr[0] == 0 and P.rowptr[-1] == P.nnz and P.rowptr.dtype == np.int32
    counts = np.diff(P.rowptr)
    assert counts.min() >= 1 and counts.max() <= c["kmax"]
    assert abs(counts.mean() - c["kmean"]) < 0.6
    for b in range(c["B"]):
        row = P.colidx[P.rowptr[b]:P.rowptr[b + 1]]
        assert (np.diff(row) > 0).all()  # sorted, no duplicates
    assert P.colidx.min() >= 0 and P.colidx.max() < 131072
    # Zipf head: label 0 is by far the most frequent
    assert np.bincount(P.colidx).argmax() == 0
    px, py = P.coo()
    assert px.dtype == torch.int64 and (np.diff(px.numpy()) >= 0).all() and len(px) == P.nnz


def test_geometric_mean_solver():
    for kmax, mean in [(8, 2.3), (20, 5.0), (30, 8.0), (50, 5.0)]:
        q = synth._geometric_q(kmax, mean)
        ks = np.arange(1, kmax + 1)
        p = q ** (ks - 1.0)
        assert abs((ks * p).sum() / p.sum() - mean) < 1e-6


def test_X_W_distributions():
    X = synth.make_X(64, 768, seed=1)
    assert torch.allclose(X.norm(dim=1), torch.ones(64), atol=1e-5)
    W = synth.make_W(4096, 768, seed=1)
    assert abs(float(W.std()) - 0.02) < 5e-4 and abs(float(W.mean())) < 1e-3
    assert torch.equal(synth.make_W(4096, 768, seed=1), W)


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "xfc_mi355x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xfc_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert len(names) >= 12
    h = lib()
    for n in names:
        assert hasattr(h, n), f"{n} declared in include/xfc_mi355x.h but not exported"
    assert set(names) == set(EXPORTS), "ctypes signatures and header disagree"
    assert h.xfc_abi_version() == 1
    assert h.xfc_strerror(0) == b"ok" and b"layout" in h.xfc_strerror(2)


def test_c_abi_argument_checks_return_codes():
    h = lib()
    one = ctypes.c_void_p(16)  # never dereferenced: every call below fails validation first
    # row-major x row-major with apply_sigmoid selects no mode
    rc = h.xfc_gemm(one, 8, 8, 8, 1, one, 8, 8, 8, 1, one, 8, 8, 8, 1, 1.0, 0.0, 1, None, 0, None)
    assert rc == 2
    # shapes that do not agree
    rc = h.xfc_gemm(one, 8, 16, 16, 1, one, 8, 8, 1, 8, one, 8, 8, 8, 1, 1.0, 0.0, 1, None, 0, None)
    assert rc == 6
    # null pointers, negative sizes
    assert h.xfc_gemm(None, 8, 8, 8, 1, one, 8, 8, 1, 8, one, 8, 8, 8, 1, 1.0, 0.0, 1, None, 0, None) == 1
    assert h.xfc_logits(one, 8, one, 8, one, 8, -1, 8, 8, None) == 1
    # misaligned leading dimension
    assert h.xfc_logits(one, 7, one, 8, one, 8, 8, 8, 8, None) == 3
    # split mode without workspace
    rc = h.xfc_gemm(one, 8, 64, 64, 1, one, 64, 8, 8, 1, one, 8, 8, 8, 1, 1.0, 0.0, 0, None, 0, None)
    assert rc == 4
    assert h.xfc_dx(one, 64, one, 8, one, 8, 8, 64, 8, 1.0, None, 0, None) == 4
    # G rows too short to hold the zeroed pad columns
    assert h.xfc_dx(one, 8, one, 8, one, 8, 8, 9, 8, 1.0, one, 1 << 30, None) == 6
    assert h.xfc_fwd_grad_workspace_bytes(1310720, 2560) > 0
    assert h.xfc_step_workspace_bytes(512, 1310720, 768, 2560) >= h.xfc_dx_workspace_bytes(512, 1310720, 768)
    # empty problems are accepted without touching the device
    assert h.xfc_logits(None, 8, None, 8, None, 8, 0, 8, 8, None) == 0
    assert h.xfc_sgd_momentum(None, None, None, 0, 0.1, 0.9, 0.0, None) == 0


def test_python_mirror_rejects_bad_arguments_without_a_gpu():
    from renee_amd import xfc_gemm

    a = torch.zeros(2, 3, 4, dtype=torch.float16)
    b = torch.zeros(4, 4, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="expected 2D tensor"):  # xfc_gemm.cpp:28-30
        xfc_gemm(a, b, b, 1.0, 0.0, True)
    with pytest.raises(RuntimeError, match="GPU"):
        xfc_gemm(b, b, b, 1.0, 0.0, True)


def test_drop_in_module_name():
    import xfc_gemm_cuda  # dl_base.py:26-32, setup.py:8

    assert callable(xfc_gemm_cuda.xfc_gemm)


def test_cosine_schedule_matches_closed_form():
    import math

    from renee_amd import cosine_schedule_with_warmup as sched

    assert sched(0, 100, 1000, 0.05) == 0.0            # lr is 0 on the first step of a warm-up
    assert abs(sched(50, 100, 1000, 0.05) - 0.025) < 1e-12
    assert abs(sched(100, 100, 1000, 0.05) - 0.05) < 1e-12
    assert abs(sched(550, 100, 1000, 0.05) - 0.025) < 1e-12
    assert abs(sched(1000, 100, 1000, 0.05)) < 1e-12
    for s in (101, 333, 999):
        p = (s - 100) / 900
        assert abs(sched(s, 100, 1000, 0.05) - 0.05 * 0.5 * (1 + math.cos(math.pi * p))) < 1e-15
    try:
        from transformers import get_cosine_schedule_with_warmup
    except Exception:
        return
    prm = torch.nn.Parameter(torch.zeros(1))
    opt = torch.optim.SGD([prm], lr=0.05)
    sch = get_cosine_schedule_with_warmup(opt, 100, 1000)
    for s in range(0, 1000, 37):
        while sch.last_epoch < s:
            opt.step()
            sch.step()
        assert abs(sch.get_last_lr()[0] - sched(s, 100, 1000, 0.05)) < 1e-12


def test_sparse_label_reader_and_batch_positives():
    from renee_amd import batch_positives, read_sparse_labels

    path = os.path.join(ROOT, "tests", "golden", "lf_amazontitles_131k_tst_first256.txt")
    rowptr, colidx, shape = read_sparse_labels(path)
    assert shape == (256, 131073) and rowptr[-1] == len(colidx) and len(colidx) > 256
    assert list(colidx[rowptr[0]:rowptr[1]]) == [42537, 43834]           # first row of the reference's file
    assert list(colidx[rowptr[1]:rowptr[2]]) == [89490, 89491, 118419, 118424]
    z = batch_positives(rowptr, colidx, [1, 0, 1])
    assert z.dtype == torch.int64 and z.shape[0] == 2
    assert z[0].tolist() == [0, 0, 0, 0, 1, 1, 2, 2, 2, 2]
    assert z[1].tolist() == [89490, 89491, 118419, 118424, 42537, 43834, 89490, 89491, 118419, 118424]
    # one rank's label columns, re-based (main.py:94-97)
    zr = batch_positives(rowptr, colidx, [1, 0], start_label=65536, end_label=131088)
    assert zr[0].tolist() == [0, 0, 0, 0] and zr[1].tolist() == [89490 - 65536, 89491 - 65536, 118419 - 65536, 118424 - 65536]


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """include/xfc_mi355x.h must be usable from C (the boundary a cgo / JNI / ctypes binding sees): it
    compiles as C99 and a C program linked against the library can call the argument checks."""
    import shutil
    import subprocess

    from renee_amd._lib import LIB_PATH

    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    hdr = os.path.join(ROOT, "include", "xfc_mi355x.h")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c", hdr],
                   check=True)
    if not os.path.exists(LIB_PATH):
        pytest.skip("library not built")
    src = tmp_path / "t.c"
    src.write_text('#include <stdio.h>\n#include "xfc_mi355x.h"\n'
                   'int main(void) {\n'
                   '  if (xfc_abi_version() != XFC_ABI_VERSION) return 1;\n'
                   '  if (xfc_logits(NULL, 8, NULL, 8, NULL, 8, 4, 4, 8, NULL) != XFC_ERR_INVALID) return 2;\n'
                   '  if (xfc_topk_workspace_bytes(4, 1000, 129) != 0) return 3;\n'
                   '  if (xfc_topk_workspace_bytes(4, 1000, 100) != (size_t)4 * 1000 * 2) return 4;\n'
                   '  printf("%s\\n", xfc_strerror(XFC_ERR_WORKSPACE));\n  return 0;\n}\n')
    exe = tmp_path / "t"
    libdir = os.path.dirname(LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                    "-L", libdir, "-l:" + os.path.basename(LIB_PATH), "-Wl,-rpath," + libdir], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out
    assert "workspace" in out.stdout.lower()
