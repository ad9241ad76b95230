"""Host side of the XFC layer step: the reference's operator interface for this
path, driving the HIP kernels through the C ABI (include/xfc_mi355x.h).

  xfc_gemm(...)            the extension function the reference imports as
                           xfc_gemm_cuda.xfc_gemm (xfc_gemm.cpp:17-40)
  XFCLayer                 the buffers GenericModel keeps for the classifier
                           (dl_base.py:175-187) and BCELossMultiNode's
                           xfc_forward / xfc_backward (dl_base.py:568-642), with
                           the optimizer step (dl_base.py:343) fused into the dW pass

PyTorch supplies device memory and the current stream; all arithmetic on the
path is done by the HIP library.
"""
from __future__ import annotations

import torch

from ._lib import check, lib


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _round_up(a: int, b: int) -> int:
    return (a + b - 1) // b * b


class _Workspace:
    """Scratch for the bare six-argument xfc_gemm: one growable byte buffer per (device, stream), so
    calls on different streams never share one.  XFCLayer does not use it: a layer owns a workspace of
    fixed size, allocated when the layer is built (the reference preallocates its large buffers for the
    same reason, dl_base.py:175-187)."""

    def __init__(self):
        self._buf = {}

    def get(self, device: torch.device, stream: int, nbytes: int) -> torch.Tensor:
        key = (device.type, device.index, int(stream))
        buf = self._buf.get(key)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
            self._buf[key] = buf
        return buf


_workspace = _Workspace()


def _require(cond: bool, msg: str, exc=RuntimeError):
    if not cond:
        raise exc(msg)


def gemm_workspace_bytes(in1_strides, in2_strides, M: int, N: int, K: int, apply_sigmoid: bool) -> int:
    """Scratch the six-argument call needs: only the row x row mode (contraction over the long axis,
    split; xfc_gemm_kernel.cu:151) uses any.  The column x row mode (dW: M = labels, N = dims) must not
    be sized by the split plan, which would ask for splits * M * N * 4 bytes (tens of gigabytes)."""
    row_row = (not apply_sigmoid) and in1_strides[1] == 1 and in2_strides[1] == 1 and in1_strides[0] != 1
    return int(lib().xfc_gemm_workspace_bytes(M, N, K)) if row_row else 0


def xfc_gemm(mat_in1: torch.Tensor, mat_in2: torch.Tensor, mat_out: torch.Tensor,
             alpha: float, beta: float, apply_sigmoid: bool) -> None:
    """Drop-in for xfc_gemm_cuda.xfc_gemm (xfc_gemm.cpp:17-23): writes mat_out in
    place; the GEMM mode follows from the strides of the views passed in
    (xfc_gemm_kernel.cu:65,113,151).  Unlike the reference, bad arguments raise
    instead of terminating the process, and dtypes/devices are checked."""
    for t in (mat_in1, mat_in2, mat_out):
        _require(t.dim() == 2, "expected 2D tensor")
        _require(t.is_cuda, "expected a GPU tensor")
    _require(mat_in1.dtype == torch.float16 and mat_in2.dtype == torch.float16,
             "mat_in1 and mat_in2 must be float16", TypeError)
    want = torch.float16 if apply_sigmoid else torch.float32
    _require(mat_out.dtype == want, f"mat_out must be {want} for apply_sigmoid={bool(apply_sigmoid)}", TypeError)
    _require(mat_in1.device == mat_in2.device == mat_out.device, "tensors must share a device")
    M, N = mat_out.shape
    K = mat_in2.shape[0]
    L = lib()
    ws_bytes = gemm_workspace_bytes(mat_in1.stride(), mat_in2.stride(), M, N, K, apply_sigmoid)
    with torch.cuda.device(mat_out.device):
        ws = _workspace.get(mat_out.device, _stream(mat_out), ws_bytes)
        rc = L.xfc_gemm(mat_in1.data_ptr(), mat_in1.shape[0], mat_in1.shape[1], mat_in1.stride(0), mat_in1.stride(1),
                        mat_in2.data_ptr(), mat_in2.shape[0], mat_in2.shape[1], mat_in2.stride(0), mat_in2.stride(1),
                        mat_out.data_ptr(), M, N, mat_out.stride(0), mat_out.stride(1),
                        float(alpha), float(beta), int(bool(apply_sigmoid)),
                        ws.data_ptr(), ws.numel(), _stream(mat_out))
    check(rc, "xfc_gemm")


def cosine_schedule_with_warmup(step: int, warmup_steps: int, total_steps: int, base_lr: float) -> float:
    """Learning rate of the XFC optimizer at `step` (dl_base.py:241,376,396-397: transformers'
    get_cosine_schedule_with_warmup, half a cosine period): linear from 0 over the warm-up, then
    base_lr * 0.5 * (1 + cos(pi * progress)).  Pass the result as `lr=` to xfc_backward / dw_update."""
    import math

    if step < warmup_steps:
        return base_lr * step / max(1, warmup_steps)
    progress = (step - warmup_steps) / max(1, total_steps - warmup_steps)
    return base_lr * max(0.0, 0.5 * (1.0 + math.cos(math.pi * progress)))


def read_sparse_labels(path: str):
    """Read a label matrix in the XC repository's sparse text format (header `rows cols`, then one line
    per row of `col:val` pairs; the format main.py:50-51 loads through pyxclib) into CSR numpy arrays
    (rowptr int64[rows+1], colidx int32[nnz], shape).  Values are ignored: labels are binary."""
    import numpy as np

    with open(path) as f:
        rows, cols = (int(v) for v in f.readline().split()[:2])
        lines = f.read().split("\n")[:rows]
    lines += [""] * (rows - len(lines))
    # one pass of numpy over the whole text instead of a Python loop over tokens
    counts = np.fromiter((ln.count(":") for ln in lines), dtype=np.int64, count=rows)
    flat = np.array(" ".join(lines).replace(":", " ").split(), dtype=np.float64)
    ids = flat[0::2].astype(np.int64)
    _require(ids.shape[0] == int(counts.sum()), "malformed label file: expected col:val pairs")
    row_of = np.repeat(np.arange(rows, dtype=np.int64), counts)
    key = np.unique(row_of * max(cols, 1) + ids)          # sorted by (row, label), duplicates dropped
    row_of, ids = key // max(cols, 1), key % max(cols, 1)
    rowptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(np.bincount(row_of, minlength=rows), out=rowptr[1:])
    return rowptr, ids.astype(np.int32), (rows, cols)


def batch_positives(rowptr, colidx, ids, start_label: int = 0, end_label: int | None = None, device=None):
    """The collator's label tensor for a batch (dl_base.py:934-936: labels[full_ids].tocoo() as a
    2 x nnz LongTensor, rows ascending), optionally restricted and re-based to one rank's label columns
    (main.py:94-97).  The result is a CPU tensor, as the collator's is, unless `device` is given;
    XFCLayer moves index tensors to its GPU itself."""
    import numpy as np

    rows, cols = [], []
    for b, i in enumerate(ids):
        c = colidx[rowptr[i]:rowptr[i + 1]]
        if end_label is not None:
            c = c[(c >= start_label) & (c < end_label)]
        elif start_label:
            c = c[c >= start_label]
        rows.append(np.full(c.shape[0], b, dtype=np.int64))
        cols.append(c.astype(np.int64) - start_label)
    z = torch.from_numpy(np.stack([np.concatenate(rows), np.concatenate(cols)])) if rows else torch.zeros(2, 0, dtype=torch.int64)
    return z if device is None else z.to(device)


def coo_to_csr(pos_x: torch.Tensor, pos_y: torch.Tensor, num_rows: int):
    """Row-sorted COO (dl_base.py:934-936) -> (rowptr int32[B+1], colidx int32[nnz]) on the same device."""
    counts = torch.bincount(pos_x.long(), minlength=num_rows)
    rowptr = torch.zeros(num_rows + 1, dtype=torch.int32, device=pos_x.device)
    rowptr[1:] = torch.cumsum(counts, 0).to(torch.int32)
    return rowptr, pos_y.to(torch.int32).contiguous()


def g_row_stride(numy: int) -> int:
    """Leading dimension (in halves) of a G buffer this library allocates: the label count rounded up to 8
    (the kernels read G in 16-byte pieces), then padded until the row stride is 256 bytes past a multiple of
    4 KB.  A batch's rows are touched side by side (128 bytes of each of 256 rows per k-step in dX); at a
    stride that is a multiple of a large power of two those accesses fall on few memory channels: measured
    at batch 1024, dX ran 17 % and dW 6 % slower at L = 2^24, the forward pass 6 % and dX 5 % slower at
    L = 1,310,720 (= 5 * 2^18), than with the stride 128-1024 bytes off."""
    ld = _round_up(numy, 8)
    if ld * 2 < 4096:   # rows shorter than 4 KB: nothing to skew
        return ld
    return ld + ((256 - ld * 2) % 4096) // 2


class XFCLayer:
    """Label matrix, momentum and scratch buffers of the classifier on one GPU,
    with the reference's xfc_forward / xfc_backward operators.

    numy is padded as main.py:76-89 does only if the caller asks (pad_to);
    any label count is accepted.  W and the momentum are fp16 and stay
    resident; G (`outsoft`, dl_base.py:176) is preallocated for max_batch rows
    with a row stride of `ldg` halves (see g_row_stride: the label count rounded
    up to 8 plus a skew that keeps the stride off large powers of two).

    Every buffer, the kernels' workspace included, is allocated here and never
    again (dl_base.py:175-187 preallocates for the same reason): a layer's calls
    can be captured into a HIP graph without a sizing pass, and two layers never
    share scratch, so they may run on two streams at once.  One layer's calls
    must stay on one stream at a time.  `max_positives` bounds the label pairs
    of one batch (default 64 per row of max_batch).

    Optimizer state.  By default W and the momentum live in fp16 only (8 bytes
    of traffic per weight and step); an update smaller than half an fp16 ulp of
    the weight it applies to is then lost to rounding.  With
    `master_weights=True` the layer keeps the reference's regime instead, an
    fp32 `xfc_weight_master` and an fp32 `momentum_buffer` (dl_base.py:185,
    main.py:178-179), and `xfc_weight` is the fp16 copy of the master that the
    GEMMs read, rewritten by the update itself (18 bytes per weight and step).
    """

    def __init__(self, numy: int, dims: int, max_batch: int, device="cuda:0", lr: float = 0.05,
                 momentum: float = 0.9, weight_decay: float = 0.0, weight: torch.Tensor | None = None,
                 seed: int = 0, max_positives: int | None = None, master_weights: bool = False):
        self.device = torch.device(device)
        _require(self.device.type == "cuda", "XFCLayer needs a GPU device")
        _require(dims % 8 == 0, "dims must be a multiple of 8")
        self.numy, self.dims, self.max_batch = int(numy), int(dims), int(max_batch)
        self.max_positives = int(max_positives) if max_positives is not None else 64 * self.max_batch
        self.lr, self.momentum, self.weight_decay = float(lr), float(momentum), float(weight_decay)
        self.ldg = g_row_stride(self.numy)
        if weight is None:
            g = torch.Generator(device=self.device)
            g.manual_seed(seed)
            weight = torch.empty(self.numy, self.dims, device=self.device, dtype=torch.float16)
            step = 1 << 20
            for r0 in range(0, self.numy, step):  # N(0, 0.02): dl_base.py:187
                r1 = min(self.numy, r0 + step)
                weight[r0:r1] = (torch.randn(r1 - r0, self.dims, generator=g, device=self.device) * 0.02).half()
            weight_in = weight
        else:
            _require(tuple(weight.shape) == (self.numy, self.dims), "weight shape")
            weight_in = weight
            weight = weight.to(device=self.device, dtype=torch.float16).contiguous()
        self.master_weights = bool(master_weights)
        if self.master_weights:
            # an fp32 weight handed in (a reference checkpoint's) is kept exactly; the fp16 copy is its rounding
            self.xfc_weight_master = weight_in.to(device=self.device, dtype=torch.float32).contiguous().clone()
            weight = self.xfc_weight_master.to(torch.float16)
            self.momentum_buffer = torch.zeros_like(self.xfc_weight_master)
        else:
            self.xfc_weight_master = None
            self.momentum_buffer = torch.zeros_like(weight)
        self.xfc_weight = weight
        self.outsoft = torch.empty(self.max_batch, self.ldg, device=self.device, dtype=torch.float16)
        self.grad_input = torch.empty(self.max_batch, self.dims, device=self.device, dtype=torch.float32)
        self.xfc_weight_grad = None  # fp32 accumulator, only under split accumulation
        self._g_live = False  # outsoft holds a G that dw_update / dw_accumulate has not consumed yet
        L = lib()
        with torch.cuda.device(self.device):
            check(L.xfc_init(), "xfc_init")
            # the largest need over every batch size up to max_batch: the per-call needs are not monotone in B
            need = max(L.xfc_layer_workspace_bytes(self.max_batch, self.numy, self.dims, self.max_positives), 256)
            self._ws = torch.empty(need, dtype=torch.uint8, device=self.device)

    # -- helpers ---------------------------------------------------------------------------
    def _x16(self, embed: torch.Tensor) -> torch.Tensor:
        _require(embed.dim() == 2 and embed.shape[1] == self.dims, "embed must be (batch, dims)")
        x = embed.to(device=self.device, dtype=torch.float16)  # dl_base.py:561
        return x if x.stride(1) == 1 and x.stride(0) % 8 == 0 else x.contiguous()

    def _g_view(self, bsz: int, out: torch.Tensor | None = None) -> torch.Tensor:
        """The G buffer of a batch: rows of `outsoft`, or a caller's `out` (the reference passes
        outsoft[0:bsz, :] itself, dl_base.py:312-313) if the kernels can use it as it is: fp16, unit
        column stride, row stride a multiple of 8 that holds the label count rounded up to 8 (the
        reference pads numy to a multiple of 16, main.py:83-87)."""
        if out is None:
            _require(bsz <= self.max_batch, "batch larger than max_batch")
            return self.outsoft[0:bsz]
        _require(out.dtype == torch.float16 and out.dim() == 2 and out.device == self.device and out.stride(1) == 1 and
                 out.shape[0] == bsz and out.shape[1] >= self.numy and out.stride(0) % 8 == 0 and
                 out.stride(0) >= _round_up(self.numy, 8) and out.data_ptr() % 16 == 0,
                 "out must be float16 (batch, numy) on the layer's device with a row stride that is a multiple of 8 "
                 "and at least numy rounded up to 8")
        return out

    def _index(self, t: torch.Tensor, dtype: torch.dtype, what: str) -> torch.Tensor:
        """An index tensor as the kernels read it: 1-D, contiguous, of `dtype`, on this layer's GPU.
        The dtype is checked, never converted (a silent int64 -> int32 pass would hide a caller's
        mistake); a tensor on another device (the collator's 'z' lives on the CPU) is copied over."""
        _require(isinstance(t, torch.Tensor) and t.dim() == 1, f"{what} must be a 1-D tensor")
        _require(t.dtype == dtype, f"{what} must be {dtype}", TypeError)
        if t.device != self.device:
            t = t.to(self.device)
        return t.contiguous()

    def _check_nnz(self, nnz: int) -> None:
        _require(nnz <= self.max_positives,
                 f"{nnz} label pairs in one batch exceed max_positives={self.max_positives}; "
                 "build the layer with a larger max_positives", ValueError)

    # -- reference operators ---------------------------------------------------------------
    def xfc_forward(self, embed: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """Logits out = embed . W^T (dl_base.py:568-573)."""
        x = self._x16(embed)
        bsz = x.shape[0]
        if out is None:
            out = self._g_view(bsz)[:, : self.numy]
        _require(out.dtype == torch.float16 and out.stride(1) == 1 and tuple(out.shape) == (bsz, self.numy)
                 and out.device == self.device,
                 "out must be float16 (batch, numy) with unit column stride on the layer's device")
        with torch.cuda.device(self.device):
            rc = lib().xfc_logits(x.data_ptr(), x.stride(0), self.xfc_weight.data_ptr(), self.dims,
                                  out.data_ptr(), out.stride(0), bsz, self.numy, self.dims, _stream(x))
        check(rc, "xfc_logits")
        return out

    def topk(self, embed: torch.Tensor, K: int = 5, numy: int | None = None, overwrite_g: bool = False):
        """Exact top-K labels per row over all labels (FullPredictor's scoring loop, dl_base.py:736-756,
        with the pad clamp of :782 when numy < the stored label count).  Returns (values fp32, indices
        int64), each (batch, K); ties go to the lower label id.  K <= 8192: up to 8 in one fused pass,
        above that (the final evaluation's K = 100, dl_base.py:817-818; torch.topk at :756) by an exact
        selection over the fp16 logits, which are written to `outsoft` as the reference's scorer does
        (dl_base.py:745).
        K > 8 therefore destroys a G that fwd_grad left in `outsoft`: between fwd_grad and the dw_update /
        dw_accumulate that consumes it the call raises unless overwrite_g=True."""
        x = self._x16(embed)
        bsz = x.shape[0]
        _require(1 <= K <= 8192 and K <= self.numy, "K must be in 1..min(8192, numy)")
        _require(bsz <= self.max_batch, "batch larger than max_batch")
        _require(K <= 8 or overwrite_g or not self._g_live,
                 "topk with K > 8 writes its logits over outsoft, which holds a G that dw_update / dw_accumulate "
                 "has not consumed yet; finish the step first or pass overwrite_g=True")
        if K > 8:
            self._g_live = False
        vals = torch.empty(bsz, K, device=self.device, dtype=torch.float32)
        inds = torch.empty(bsz, K, device=self.device, dtype=torch.int64)
        L = lib()
        ws = self.outsoft if K > 8 else self._ws
        with torch.cuda.device(self.device):
            rc = L.xfc_topk(x.data_ptr(), x.stride(0), self.xfc_weight.data_ptr(), self.dims, bsz, self.numy,
                            self.dims, self.numy if numy is None else int(numy), int(K), vals.data_ptr(),
                            inds.data_ptr(), ws.data_ptr(), ws.numel() * ws.element_size(), _stream(x))
        check(rc, "xfc_topk")
        return vals, inds

    def fwd_grad(self, embed, pos_x=None, pos_y=None, rowptr=None, colidx=None,
                 loss_out: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
        """G = sigmoid(embed . W^T) - Y into outsoft (dl_base.py:591-594); returns the (batch, numy) view.
        With loss_out (a one-element float32 tensor) the summed BCE loss of the batch
        (dl_base.py:578-583) is produced by the same pass."""
        if loss_out is not None:
            _require(loss_out.dtype == torch.float32 and loss_out.numel() == 1 and loss_out.device == self.device,
                     "loss_out must be a one-element float32 tensor on the layer's device")
        lp = None if loss_out is None else loss_out.data_ptr()
        x = self._x16(embed)
        bsz = x.shape[0]
        G = self._g_view(bsz, out)
        ldg = G.stride(0)
        L = lib()
        csr = rowptr is not None
        ws = self._ws
        # every index tensor is validated and brought to this GPU before anything is launched
        if csr:
            rowptr = self._index(rowptr, torch.int32, "rowptr")
            colidx = self._index(colidx, torch.int32, "colidx")
            _require(rowptr.numel() == bsz + 1, "rowptr must have batch+1 entries")
            nnz = int(colidx.numel())
        else:
            nnz = 0 if pos_x is None else int(pos_x.numel())
            if nnz:
                pos_x = self._index(pos_x, torch.int64, "pos_x")
                pos_y = self._index(pos_y, torch.int64, "pos_y")
                _require(pos_x.numel() == pos_y.numel(), "pos_x / pos_y length")
        self._check_nnz(nnz)
        with torch.cuda.device(self.device):
            if csr:
                rc = L.xfc_fwd_grad_csr(x.data_ptr(), x.stride(0), self.xfc_weight.data_ptr(), self.dims,
                                        rowptr.data_ptr(), colidx.data_ptr(), G.data_ptr(), ldg,
                                        bsz, self.numy, self.dims, nnz, lp, ws.data_ptr(), ws.numel(), _stream(x))
            else:
                rc = L.xfc_fwd_grad_coo(x.data_ptr(), x.stride(0), self.xfc_weight.data_ptr(), self.dims,
                                        pos_x.data_ptr() if nnz else None, pos_y.data_ptr() if nnz else None, nnz,
                                        G.data_ptr(), ldg, bsz, self.numy, self.dims, lp,
                                        ws.data_ptr(), ws.numel(), _stream(x))
        check(rc, "xfc_fwd_grad")
        if out is None:
            self._g_live = True
        return G[:, : self.numy]

    def dx(self, bsz: int, grad_input: torch.Tensor | None = None, scale: float = 1.0,
           out: torch.Tensor | None = None) -> torch.Tensor:
        """grad_input = scale * G . W with W before the update (dl_base.py:602-608)."""
        if grad_input is None:
            grad_input = self.grad_input[0:bsz]
        _require(grad_input.dtype == torch.float32 and grad_input.stride(1) == 1 and
                 tuple(grad_input.shape) == (bsz, self.dims) and grad_input.device == self.device,
                 "grad_input must be float32 (batch, dims) on the layer's device")
        L = lib()
        G = self._g_view(bsz, out)
        ws = self._ws
        with torch.cuda.device(self.device):
            rc = L.xfc_dx(G.data_ptr(), G.stride(0), self.xfc_weight.data_ptr(), self.dims, grad_input.data_ptr(),
                          grad_input.stride(0), bsz, self.numy, self.dims, float(scale),
                          ws.data_ptr(), ws.numel(), _stream(G))
        check(rc, "xfc_dx")
        return grad_input

    def dw_update(self, embed, dW_out: torch.Tensor | None = None, lr: float | None = None,
                  out: torch.Tensor | None = None) -> None:
        """dW = G^T . embed fused with M = mu*M + dW + wd*W ; W -= lr*M (dl_base.py:620-634 + :343)."""
        x = self._x16(embed)
        bsz = x.shape[0]
        G = self._g_view(bsz, out)
        ldg = G.stride(0)
        if dW_out is not None:
            _require(dW_out.dtype == torch.float32 and dW_out.is_contiguous() and dW_out.device == self.device and
                     tuple(dW_out.shape) == (self.numy, self.dims),
                     "dW_out must be contiguous float32 (numy, dims) on the layer's device")
        if self.master_weights:
            with torch.cuda.device(self.device):
                rc = lib().xfc_dw_update_master(G.data_ptr(), ldg, x.data_ptr(), x.stride(0),
                                                self.xfc_weight_master.data_ptr(), self.dims,
                                                self.momentum_buffer.data_ptr(), self.dims,
                                                self.xfc_weight.data_ptr(), self.dims, bsz, self.numy, self.dims,
                                                self.lr if lr is None else float(lr), self.momentum, self.weight_decay,
                                                None if dW_out is None else dW_out.data_ptr(), self.dims, _stream(x))
            check(rc, "xfc_dw_update_master")
            self._g_live = self._g_live and out is not None
            return
        with torch.cuda.device(self.device):
            rc = lib().xfc_dw_update(G.data_ptr(), ldg, x.data_ptr(), x.stride(0),
                                     self.xfc_weight.data_ptr(), self.dims, self.momentum_buffer.data_ptr(), self.dims,
                                     bsz, self.numy, self.dims, self.lr if lr is None else float(lr), self.momentum,
                                     self.weight_decay, None if dW_out is None else dW_out.data_ptr(), self.dims,
                                     _stream(x))
        check(rc, "xfc_dw_update")
        self._g_live = self._g_live and out is not None

    def dw_accumulate(self, embed, out: torch.Tensor | None = None) -> None:
        """xfc_weight.grad (+)= G^T . embed for one micro-batch (dl_base.py:620-633)."""
        x = self._x16(embed)
        bsz = x.shape[0]
        G = self._g_view(bsz, out)
        first = self.xfc_weight_grad is None
        if first:
            self.xfc_weight_grad = torch.empty(self.numy, self.dims, device=self.device, dtype=torch.float32)
        with torch.cuda.device(self.device):
            rc = lib().xfc_dw(G.data_ptr(), G.stride(0), x.data_ptr(), x.stride(0), self.xfc_weight_grad.data_ptr(),
                              self.dims, bsz, self.numy, self.dims, 0.0 if first else 1.0, _stream(x))
        check(rc, "xfc_dw")
        self._g_live = self._g_live and out is not None

    def optimizer_step(self, lr: float | None = None) -> None:
        """SGD-momentum on the accumulated fp32 grad, then drop it (dl_base.py:343-344)."""
        _require(self.xfc_weight_grad is not None, "no accumulated gradient")
        if self.master_weights:
            with torch.cuda.device(self.device):
                rc = lib().xfc_sgd_momentum_master(self.xfc_weight_master.data_ptr(), self.momentum_buffer.data_ptr(),
                                                   self.xfc_weight.data_ptr(), self.xfc_weight_grad.data_ptr(),
                                                   self.numy * self.dims, self.lr if lr is None else float(lr),
                                                   self.momentum, self.weight_decay, _stream(self.xfc_weight))
            check(rc, "xfc_sgd_momentum_master")
            self.xfc_weight_grad = None
            return
        with torch.cuda.device(self.device):
            rc = lib().xfc_sgd_momentum(self.xfc_weight.data_ptr(), self.momentum_buffer.data_ptr(),
                                        self.xfc_weight_grad.data_ptr(), self.numy * self.dims,
                                        self.lr if lr is None else float(lr), self.momentum, self.weight_decay,
                                        _stream(self.xfc_weight))
        check(rc, "xfc_sgd_momentum")
        self.xfc_weight_grad = None

    # -- checkpoint payload (dl_base.py:412-446 keeps xfc_weight and the optimizer state per rank) ------
    def state_dict(self) -> dict:
        """W and the momentum as CPU tensors (fp16, or the fp32 master and momentum when the layer keeps
        them) plus the hyper-parameters, for a checkpoint."""
        w = self.xfc_weight_master if self.master_weights else self.xfc_weight
        return {"xfc_weight": w.detach().cpu(), "momentum_buffer": self.momentum_buffer.detach().cpu(),
                "numy": self.numy, "dims": self.dims, "lr": self.lr, "momentum": self.momentum,
                "weight_decay": self.weight_decay}

    def load_state_dict(self, state: dict, optimizer_state: dict | None = None) -> None:
        """Restore from state_dict().  A reference checkpoint is accepted too: its fp32 `xfc_weight`
        (dl_base.py:420) is rounded to fp16 once, and `optimizer_state` may be the reference's
        `xfc_optimizer_state_dict` (dl_base.py:424; torch's optimizer layout, {'state': {0:
        {'momentum_buffer': fp32 L x d}}, 'param_groups': [...]}), whose momentum buffer is rounded to
        fp16 the same way.  Without any momentum the buffer starts from zero, as the optimizer's
        first step does."""
        w = state["xfc_weight"]
        _require(tuple(w.shape) == (self.numy, self.dims), "checkpoint shape does not match this layer")
        if self.master_weights:
            self.xfc_weight_master.copy_(w.to(device=self.device, dtype=torch.float32))
            self.xfc_weight.copy_(self.xfc_weight_master)
        else:
            self.xfc_weight.copy_(w.to(device=self.device, dtype=torch.float16))
        m = state.get("momentum_buffer")
        if m is None and optimizer_state is not None:
            per_param = list(optimizer_state.get("state", {}).values())
            _require(len(per_param) <= 1, "the XFC optimizer holds one parameter (dl_base.py:222-238)")
            if per_param:
                m = per_param[0].get("momentum_buffer")
        if m is None:
            self.momentum_buffer.zero_()
        else:
            _require(tuple(m.shape) == (self.numy, self.dims), "momentum buffer shape does not match this layer")
            self.momentum_buffer.copy_(m.to(device=self.device, dtype=self.momentum_buffer.dtype))
        for k in ("lr", "momentum", "weight_decay"):
            if k in state:
                setattr(self, k, float(state[k]))
        self.xfc_weight_grad = None

    def xfc_backward(self, embed_out, pos_x, pos_y, grad_input=None, scale: float = 1.0,
                     accumulate: bool = False, lr: float | None = None) -> torch.Tensor:
        """One batch (or micro-batch) of dl_base.py:576-642 under --noloss: G, then
        grad_input, then dW.  With accumulate=False the optimizer step is fused
        into the dW pass; with accumulate=True dW is added to the fp32 grad and
        optimizer_step() finishes the step."""
        bsz = embed_out.shape[0]
        self.fwd_grad(embed_out, pos_x, pos_y)
        gi = self.dx(bsz, grad_input, scale)
        if accumulate:
            self.dw_accumulate(embed_out)
        else:
            self.dw_update(embed_out, lr=lr)
        return gi

    def step_csr(self, embed, rowptr, colidx, scale: float = 1.0, lr: float | None = None) -> torch.Tensor:
        """The whole step through the single C entry point xfc_step_csr (with fp32 master weights: the
        same three passes through their own entry points, the update being xfc_dw_update_master)."""
        if self.master_weights:
            self.fwd_grad(embed, rowptr=rowptr, colidx=colidx)
            gi = self.dx(embed.shape[0], None, scale)
            self.dw_update(embed, lr=lr)
            return gi
        x = self._x16(embed)
        bsz = x.shape[0]
        G = self._g_view(bsz)
        gi = self.grad_input[0:bsz]
        L = lib()
        rowptr = self._index(rowptr, torch.int32, "rowptr")
        colidx = self._index(colidx, torch.int32, "colidx")
        _require(rowptr.numel() == bsz + 1, "rowptr must have batch+1 entries")
        nnz = int(colidx.numel())
        self._check_nnz(nnz)
        ws = self._ws
        with torch.cuda.device(self.device):
            rc = L.xfc_step_csr(x.data_ptr(), x.stride(0), self.xfc_weight.data_ptr(), self.dims,
                                self.momentum_buffer.data_ptr(), self.dims, rowptr.data_ptr(), colidx.data_ptr(), nnz,
                                G.data_ptr(), self.ldg, gi.data_ptr(), self.dims, bsz, self.numy, self.dims,
                                self.lr if lr is None else float(lr), self.momentum, self.weight_decay, float(scale),
                                ws.data_ptr(), ws.numel(), _stream(x))
        check(rc, "xfc_step_csr")
        return gi
