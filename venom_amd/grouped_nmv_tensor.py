"""Python side of the V:N:M format for the end-to-end path: the magnitude sparsifier and the
tensor container that `SrnmSpmm` feeds to `spatha.spmm`.

Same names and attribute meaning as the reference's end2end/grouped_nmv_tensor.py
(`nm_vector_mask_sparsify` :746-779, `SrNMTensor` :677-744), but nothing is compiled at run
time: all work is done by libspatha.so through the C ABI."""
import numpy as np
import torch

from . import format as F


def round_up(x, y):
    return -(-x // y) * y


def nm_vector_mask_sparsify(tensor, n, m, tileM, threads=0, gpu=None, exact_ties=True):
    """Per tileM x m block keep the 4 columns with the largest sum of per-row top-n magnitudes,
    per row the n largest of those.  Returns (masks int32 [rows, cols], columns int32 flat), both
    on the CPU, like the reference.  gpu: search the column subsets on the GPU (default: when the
    tensor lives there); the result is the same bit for bit.  exact_ties=False (with gpu): equal magnitudes are
    resolved towards the lower column instead of through the reference's history-dependent order, which avoids a
    sequential replay of the whole search whenever such a tie occurs (common for fp16 weights)."""
    if tensor.dim() != 2:
        raise NotImplementedError("Only support layers of dimension 2")
    if gpu is None:
        gpu = tensor.is_cuda
    mag = tensor.detach().to(dtype=torch.float32, device="cpu").abs().contiguous().numpy()
    if gpu:
        dev = tensor.device if tensor.is_cuda else torch.device("cuda:0")
        with torch.cuda.device(dev):
            masks, columns = F.select_columns(mag, n, m, tileM, threads=threads, gpu=True,
                                              stream=torch.cuda.current_stream(dev).cuda_stream, exact_ties=exact_ties)
    else:
        masks, columns = F.select_columns(mag, n, m, tileM, threads=threads)
    return torch.from_numpy(masks), torch.from_numpy(columns)


class SrNMTensor:
    """A weight matrix in V:N:M form.  values fp16 / columns int32 / metadata int32 live on
    `device`; nrows, ncols, nnz as in the reference.  `to_dense()` decodes for real (the
    reference returns a tensor of ones there)."""

    def __init__(self, n_, m_, tileM_, dense_, mask_, columns_, device_):
        self.n, self.m, self.tileM = n_, m_, tileM_
        self.device = device_
        self.nrows, self.ncols = dense_.shape
        geo = F.geometry(self.nrows, self.ncols, n_, m_, tileM_)
        self.nnz = self.nrows * geo.ksp
        dense32 = dense_.detach().to(dtype=torch.float32, device="cpu").contiguous().numpy()
        mask32 = mask_.detach().to(device="cpu").to(torch.int32).contiguous().numpy()
        cols = columns_.detach().to(device="cpu").to(torch.int32).contiguous().numpy().reshape(-1)
        if cols.size != geo.n_columns:
            # callers that build column-loc without the padding groups of Ksp (the reference's
            # fixed-pattern sparsifier does) get them appended as zeros
            per_block = cols.size // (self.nrows // tileM_)
            full = np.zeros((self.nrows // tileM_, geo.n_columns // (self.nrows // tileM_)), np.int32)
            full[:, :per_block] = cols.reshape(self.nrows // tileM_, per_block)
            cols = full.reshape(-1)
        # the encoder runs in fp32 and the values are rounded to fp16 afterwards, as in the reference
        values32, metadata = F.encode(dense32, cols.astype(np.uint32), n_, m_, tileM_, mask=mask32)
        self.values = torch.from_numpy(values32).to(device=device_).half()
        self.metadata = torch.from_numpy(metadata.view(np.int32)).to(device=device_)
        self.columns = torch.from_numpy(cols).to(device=device_)

    def to_dense(self):
        dense = F.decode(self.values.float().cpu().numpy(), self.metadata.cpu().numpy().view(np.uint32),
                         self.columns.cpu().numpy().astype(np.uint32), self.nrows, self.ncols, self.n, self.m, self.tileM)
        return torch.from_numpy(dense).to(device=self.device).half()
