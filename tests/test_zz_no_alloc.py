"""xfc_fwd_grad_csr_static (the entry point that allocates nothing: its label buckets live in a fixed
array inside the library's device image) against xfc_fwd_grad_csr with a caller workspace, through
the C ABI: bit-identical G and loss, on two calls in a row, the second with a smaller input, so that
whatever the first call left in the shared array must not leak into the second."""
import pytest
import torch

from renee_amd import synth
from renee_amd._lib import check, lib

pytestmark = pytest.mark.gpu


def _both(dev, B, L, d, kmax, kmean, seed, with_loss):
    h = lib()
    check(h.xfc_init(), "xfc_init")
    X = synth.make_X(B, d, seed).half().to(dev)
    W = synth.make_W(L, d, seed).half().to(dev)
    P = synth.make_positives(B, L, kmax, kmean, 1.0, seed)
    rp, ci = torch.from_numpy(P.rowptr).to(dev), torch.from_numpy(P.colidx).to(dev)
    ldg = (L + 7) // 8 * 8
    st = torch.cuda.current_stream().cuda_stream
    out = []
    for static in (False, True):
        G = torch.full((B, ldg), float("nan"), dtype=torch.float16, device=dev)
        loss = torch.full((1,), float("nan"), dtype=torch.float32, device=dev)
        lp = loss.data_ptr() if with_loss else None
        print(f"no-alloc parity: static={static} B={B} L={L} d={d} nnz={P.nnz} loss={with_loss}", flush=True)
        if static:
            rc = h.xfc_fwd_grad_csr_static(X.data_ptr(), d, W.data_ptr(), d, rp.data_ptr(), ci.data_ptr(),
                                           G.data_ptr(), ldg, B, L, d, P.nnz, lp, st)
        else:
            ws = torch.empty(h.xfc_fwd_grad_workspace_bytes(L, P.nnz), dtype=torch.uint8, device=dev)
            rc = h.xfc_fwd_grad_csr(X.data_ptr(), d, W.data_ptr(), d, rp.data_ptr(), ci.data_ptr(),
                                    G.data_ptr(), ldg, B, L, d, P.nnz, lp, ws.data_ptr(), ws.numel(), st)
        check(rc, "xfc_fwd_grad_csr(_static)")
        torch.cuda.synchronize()
        out.append((G, loss))
    (G0, l0), (G1, l1) = out
    assert not bool(torch.isnan(G0).any())
    assert torch.equal(G0, G1)
    assert int((G0[:, :L] < 0).sum()) == P.nnz   # the positives, and only they, are below zero
    if with_loss:
        assert torch.equal(l0, l1) and bool(torch.isfinite(l0).all())


def test_static_entry_point_matches_workspace_entry_point(dev):
    # two calls in a row on the same device's array: a larger problem, then a smaller one
    _both(dev, 300, 70001, 128, 20, 6.0, seed=31, with_loss=True)
    _both(dev, 40, 1000, 64, 4, 1.5, seed=32, with_loss=False)


def test_static_entry_point_rejects_what_does_not_fit(dev):
    h = lib()
    t = torch.zeros(64, dtype=torch.float16, device=dev)
    i32 = torch.zeros(9, dtype=torch.int32, device=dev)
    # 4 M positives need 32 MB of bucket entries: beyond the fixed array, refused before any launch
    rc = h.xfc_fwd_grad_csr_static(t.data_ptr(), 8, t.data_ptr(), 8, i32.data_ptr(), i32.data_ptr(), t.data_ptr(), 8,
                                   8, 8, 8, 4_000_000, None, torch.cuda.current_stream().cuda_stream)
    assert rc == 7 and b"capacity" in h.xfc_strerror(rc)
