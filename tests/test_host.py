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
                   '  if (xfc_topk_workspace_bytes(4, 10000, 8193) != 0) return 3;\n'
                   '  if (xfc_topk_workspace_bytes(4, 1000, 100) != (size_t)4 * 1000 * 2) return 4;\n'
                   '  printf("%s\\n", xfc_strerror(XFC_ERR_WORKSPACE));\n  return 0;\n}\n')
    exe = tmp_path / "t"
    libdir = os.path.dirname(LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                    "-L", libdir, "-l:" + os.path.basename(LIB_PATH), "-Wl,-rpath," + libdir], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out
    assert "workspace" in out.stdout.lower()


def test_gemm_workspace_is_requested_only_for_the_split_mode():
    """The column x row call the reference makes for dW (out.t(), embed -> L x d, dl_base.py:623) uses
    no workspace; sizing it by the split plan would ask for tens of gigabytes at the headline shape."""
    from renee_amd.xfc import gemm_workspace_bytes

    L, B, d = 1310720, 512, 768
    assert gemm_workspace_bytes((1, L), (d, 1), L, d, B, False) == 0          # dW: G^T view x X
    assert gemm_workspace_bytes((d, 1), (1, d), B, L, d, True) == 0           # sigmoid: X x W^T view
    need = gemm_workspace_bytes((L, 1), (d, 1), B, d, L, False)               # dX: G x W, split over labels
    assert need == lib().xfc_gemm_workspace_bytes(B, d, L) and 0 < need < (1 << 30)


def test_empty_batch_is_accepted_without_touching_the_device():
    h = lib()
    one = ctypes.c_void_p(16)
    assert h.xfc_dw_update(one, 8, one, 8, one, 8, one, 8, 0, 8, 8, 0.1, 0.9, 0.0, None, 0, None) == 0
    assert h.xfc_dw(one, 8, one, 8, one, 8, 0, 8, 8, 1.0, None) == 0
    assert h.xfc_dw(one, 8, one, 8, one, 8, 0, 8, 8, 0.0, None) == 1


# ---------------------------------------------------------------------------------------------------
# The main loop's hand-counted waits (renee_amd/csrc/pipe_core.hpp, PipeCore::run): a model of what the
# hardware guarantees, run over the schedule the code issues, for every instantiation in the kernels.
#   * a wave's global->LDS fetches retire in issue order; other vector-memory operations (an epilogue's
#     loads and stores) share the counter and may retire at any time relative to the fetches;
#   * s_waitcnt vmcnt(N) returns once at most N operations are outstanding, whichever they are;
#   * after the s_barrier that follows it, what one wave knows about its own fetches holds for all.
# Checked: no stage is read before its fetches are certain to have landed, and no slot is refilled
# before every wave is past its last read of the stage it held.
# ---------------------------------------------------------------------------------------------------
def _pipecore_instantiations():
    import re

    src = open(os.path.join(ROOT, "renee_amd", "csrc", "xfc_kernels.hip")).read()
    found = {}
    for name, args in re.findall(r"using\s+(\w+)\s*=\s*PipeCore<([^>]*)>", src):
        v = [a.strip() for a in args.split(",")]
        bm, bn, bk, wm, wn, stages = (int(x) for x in v[:6])
        fetch_waves = int(v[11]) if len(v) > 11 and int(v[11]) > 0 else wm * wn   # waves that issue the fetches
        loads = (bm * bk // 8 + bn * bk // 8) // (64 * fetch_waves)               # per fetching wave
        found[name] = (stages, loads)
    return found


def _simulate_ring(stages, loads, item_stages, epilogue_ops, slack=0):
    """Walks PipeCore::run's schedule for one wave.  Returns a list of error strings (empty = safe)."""
    errors = []
    total = sum(item_stages)
    outstanding = []            # issue-ordered: ('f', stage) per fetch instruction, ('o',) per epilogue op
    landed = set()              # fetch stages certain to have landed (for every wave, once a barrier passed)
    released = set()            # stages every wave has finished reading
    issued = 0

    def issue_one():
        nonlocal issued
        s = issued              # stages past the end are the zero-block fetches that keep the count constant
        prev = s - stages       # the stage that lived in this slot
        if prev >= 0 and prev < total and prev not in released:
            errors.append(f"slot of stage {prev} refilled with stage {s} before all waves were past reading it")
        outstanding.extend([("f", s)] * loads)
        issued += 1

    def wait_vmcnt_barrier(n):
        # adversary: epilogue operations retire first, then the oldest fetches, until at most n remain
        nonlocal outstanding
        excess = len(outstanding) - n
        if excess > 0:
            others = [i for i, op in enumerate(outstanding) if op[0] == "o"][:excess]
            keep = [op for i, op in enumerate(outstanding) if i not in set(others)]
            excess -= len(others)
            outstanding = keep[max(0, excess):]
        pending = {op[1] for op in outstanding if op[0] == "f"}
        for s in range(issued):
            if s not in pending:
                landed.add(s)

    def read(stage):
        if stage < total and stage not in landed:
            errors.append(f"stage {stage} read before its fetches are known to have landed")

    for _ in range(stages - 1):
        issue_one()
    wait_vmcnt_barrier((stages - 2) * loads + slack)
    issue_one()
    read(0)
    c = 0
    drain_all = False
    for nk in item_stages:
        for _ in range(nk):
            read(c)                                  # the sub-steps' fragment reads of stage c
            wait_vmcnt_barrier(0 if drain_all else (stages - 2) * loads + slack)
            drain_all = False
            released.add(c)                          # every wave's reads of stage c precede its barrier arrival
            issue_one()                              # stage c + STAGES into the slot of stage c
            read(c + 1)                              # first fragments of the next stage
            c += 1
        outstanding.extend([("o",)] * epilogue_ops)  # the epilogue's own loads and stores
        drain_all = True
    return errors


def test_main_loop_wait_counts_never_expose_a_stage_in_flight():
    src = open(os.path.join(ROOT, "renee_amd", "csrc", "pipe_core.hpp")).read()
    # the model below mirrors these statements of PipeCore::run; if they change, so must the model
    assert src.count("wait_vmcnt_barrier<(STAGES - 2) * LOADS_PER_STAGE>()") == 1
    assert src.count("wait_lds_vmcnt_barrier<(STAGES - 2) * LOADS_PER_STAGE>()") == 1
    assert "if (drain_all) { wait_lds_vmcnt_barrier<0>(); drain_all = false; }" in src
    assert "for (int s = 0; s < STAGES - 1; ++s) issue_one();" in src
    inst = _pipecore_instantiations()
    assert {"FwdCore", "DxCore", "DwCore"} <= set(inst)
    shapes = dict(inst)
    shapes.update({"three_slots": (3, 8), "four_slots": (4, 4), "five_slots": (5, 2)})  # deeper rings the template allows
    for name, (stages, loads) in shapes.items():
        assert stages >= 2 and (stages - 1) * loads < 64, name   # vmcnt is a 6-bit counter
        for items in ([1], [1, 1, 1], [3, 1, 2], [12], [2] * 7, [16, 16]):
            for ep in (0, 3, 40):
                assert _simulate_ring(stages, loads, items, ep) == [], (name, items, ep)
    # the model does catch a wait that is one stage too permissive
    for stages, loads in ((3, 8), (4, 4)):
        assert _simulate_ring(stages, loads, [12], 0, slack=loads) != []


def test_g_row_stride_is_skewed_off_powers_of_two():
    from renee_amd.xfc import g_row_stride

    for L in (1310720, 2812281, 16777216, 131072, 131073, 4097):
        ld = g_row_stride(L)
        assert ld % 8 == 0 and ld >= (L + 7) // 8 * 8 and ld - L < 2048 + 8
        assert (ld * 2) % 4096 == 256
    assert g_row_stride(9) == 16 and g_row_stride(1000) == 1000


def test_layer_workspace_covers_every_batch_size_up_to_max_batch():
    """The per-call workspace needs are not monotone in the batch size (the dX split plan and the top-K label
    groups both grow when the batch shrinks past a row-tile boundary); a layer serves any batch up to max_batch
    on buffers allocated once (dl_base.py:175-187, :318-340), so its workspace must cover the largest need."""
    h = lib()
    saw_non_monotone = False
    for L in (70001, 1310720):
        for dims in (8, 16, 32, 64, 768):
            for max_batch in (300, 384, 512, 1024):
                nnz = 64 * max_batch
                have = h.xfc_layer_workspace_bytes(max_batch, L, dims, nnz)
                at_max = max(h.xfc_step_workspace_bytes(max_batch, L, dims, nnz), h.xfc_topk_workspace_bytes(max_batch, L, 8))
                for b in range(1, max_batch + 1):
                    need = max(h.xfc_step_workspace_bytes(b, L, dims, nnz), h.xfc_topk_workspace_bytes(b, L, 8))
                    assert need <= have, (L, dims, max_batch, b, need, have)
                    saw_non_monotone |= need > at_max
    assert saw_non_monotone  # the case this function exists for does occur in the sweep
    # K below 8 never needs more than K = 8
    assert h.xfc_topk_workspace_bytes(256, 70001, 5) <= h.xfc_layer_workspace_bytes(300, 70001, 16, 64 * 300)
