"""Writes the golden vectors under tests/golden/ by running the reference's own
Python host code (end2end/grouped_nmv_tensor.py: the magnitude selector, the
mask-driven dense->V:N:M encoder and the V:N:M->dense decoder).

Runs only in the development container, where /root/reference is mounted; the
test-suite reads the committed .npz files and never imports the reference.

Why these three functions get vectors: the storage layout (which slot of
`values` / which bits of `metadata` a (row, group, kept-entry) lands in) is a
convention of the reference, not something mathematics fixes, and the selector's
choice among equal-magnitude candidates depends on the persistent permutation
state of its std::partial_sort calls.  Neither can be pinned by an invariant.

Usage:  cd <an empty scratch directory> && python <repository>/tests/golden/make_golden.py
(the reference JIT-compiles its embedded C++ into ./.compile_cache of the cwd).
"""
import os
import sys

import numpy as np
import torch

REF = "/root/reference/end2end"
OUT = os.path.dirname(os.path.abspath(__file__))


def main():
    sys.path.insert(0, REF)
    import grouped_nmv_tensor as ref  # noqa: E402  (reference code, read-only)

    rng = np.random.default_rng(20240607)
    cases = []
    kind_of = {}

    def add(name, rows, cols, n, m, v, kind):
        if kind == "gauss":
            d = rng.standard_normal((rows, cols)).astype(np.float32)
        elif kind == "ties":      # small integers: many equal magnitudes and exact zeros
            d = rng.integers(-3, 4, size=(rows, cols)).astype(np.float32)
        elif kind == "zeros":     # some all-zero V x m blocks
            d = rng.standard_normal((rows, cols)).astype(np.float32)
            d[:, : 2 * m] = 0.0
        else:
            raise ValueError(kind)
        cases.append((name, d, n, m, v))
        kind_of[name] = kind

    add("g_64x32_m8_v32", 64, 32, 2, 8, 32, "gauss")
    add("t_32x64_m16_v32", 32, 64, 2, 16, 32, "ties")
    add("t_64x64_m8_v64", 64, 64, 2, 8, 64, "ties")
    add("g_128x48_m8_v64", 128, 48, 2, 8, 64, "gauss")      # Ksp 12 -> 16: padding groups
    add("g_64x32_m4_v32", 64, 32, 2, 4, 32, "gauss")        # plain 2:4
    add("g_32x64_m32_v32", 32, 64, 2, 32, 32, "gauss")
    add("z_64x64_m8_v32", 64, 64, 2, 8, 32, "zeros")
    add("g_64x34_m8_v32", 64, 34, 2, 8, 32, "gauss")        # cols % m == 2
    add("t_64x35_m8_v32", 64, 35, 2, 8, 32, "ties")         # cols % m == 3
    add("g_64x38_m8_v32", 64, 38, 2, 8, 32, "gauss")        # cols % m == 6
    add("g_128x128_m8_v128", 128, 128, 2, 8, 128, "gauss")
    add("g_64x256_m8_v32", 64, 256, 2, 8, 32, "gauss")      # Ksp 64: eight metadata k-tiles
    add("t_96x160_m16_v32", 96, 160, 2, 16, 32, "ties")      # Ksp 20 -> 32

    for name, d, n, m, v in cases:
        t = torch.from_numpy(d.copy())
        masks, columns = ref.nm_vector_mask_sparsify(t, n, m, v)
        sp = ref.SrNMTensor(n, m, v, t * masks.to(torch.float32), masks, columns.clone(), "cpu")
        # the reference keeps fp32 values until .half(); redo the encode to keep the fp32 array
        rows, cols = d.shape
        ksp = ref.round_up((ref.round_up(cols, m) / m) * n, 16)
        values32 = torch.zeros(rows * ksp, dtype=torch.float32)
        meta = torch.zeros(rows // 2 * ksp // 8, dtype=torch.int32)
        enc = ref.to_sparse_sr_nm((rows, cols), torch.float32, n, m, v)
        pruned = (t * masks.to(torch.float32)).contiguous()
        enc(pruned.data_ptr(), masks.data_ptr(), values32.data_ptr(), columns.data_ptr(), meta.data_ptr())
        # A V x m block that is entirely zero gets no kept entry at all; the encoder then
        # emits whatever its never-initialised scratch arrays hold, so two runs differ.
        # Those cases keep only the selector outputs.
        defined = bool(torch.equal(values32.half(), sp.values) and torch.equal(meta, sp.metadata))
        assert defined or kind_of[name] == "zeros"
        dec = ref.to_dense((rows, cols), torch.float32, n, m, v)
        back = torch.zeros((rows, cols), dtype=torch.float32)
        dec(back.data_ptr(), values32.data_ptr(), columns.data_ptr(), meta.data_ptr())
        np.savez_compressed(
            os.path.join(OUT, f"vnm_{name}.npz"),
            dense=d, n=n, m=m, v=v, ksp=int(ksp), encode_defined=(kind_of[name] != "zeros"),
            masks=masks.numpy(), columns=columns.numpy(),
            values=values32.numpy(), metadata=meta.numpy(), decoded=back.numpy(),
        )
        print(name, "ksp", int(ksp), "kept", int(masks.sum()), "roundtrip", bool(torch.equal(back, pruned)))

    # The fixed pattern the BERT harness feeds the encoder (bert_pytorch.py:62-75):
    # column-loc {0,1,2,3} in every group, mask [1,0,1,0,0,...].
    for name, rows, cols, m, v in (("fixed_128x64_m8_v64", 128, 64, 8, 64), ("fixed_64x128_m16_v32", 64, 128, 16, 32)):
        n = 2
        d = rng.standard_normal((rows, cols)).astype(np.float32)
        t = torch.from_numpy(d.copy())
        columns = torch.zeros(rows // v, cols // m * 4, dtype=torch.int32)
        columns = columns.reshape((-1, 4)) + torch.tensor([0, 1, 2, 3], dtype=torch.int32)
        columns = columns.reshape((rows // v, cols // m * 4)).contiguous()
        mk = torch.cat((torch.tensor([1, 0, 1, 0]), torch.zeros(m - 4)), 0)
        mask = (torch.zeros(t.shape).reshape(-1, v, m) + mk).reshape(t.shape)
        ksp = ref.round_up((ref.round_up(cols, m) / m) * n, 16)
        # the harness passes a float mask; the encoder reads it as int32, so hand it int32 here
        mask_i = mask.to(torch.int32).contiguous()
        values32 = torch.zeros(rows * ksp, dtype=torch.float32)
        meta = torch.zeros(rows // 2 * ksp // 8, dtype=torch.int32)
        enc = ref.to_sparse_sr_nm((rows, cols), torch.float32, n, m, v)
        flat_cols = columns.reshape(-1).contiguous()
        enc(t.data_ptr(), mask_i.data_ptr(), values32.data_ptr(), flat_cols.data_ptr(), meta.data_ptr())
        dec = ref.to_dense((rows, cols), torch.float32, n, m, v)
        back = torch.zeros((rows, cols), dtype=torch.float32)
        dec(back.data_ptr(), values32.data_ptr(), flat_cols.data_ptr(), meta.data_ptr())
        np.savez_compressed(
            os.path.join(OUT, f"vnm_{name}.npz"),
            dense=d, n=n, m=m, v=v, ksp=int(ksp), encode_defined=True,
            masks=mask_i.numpy(), columns=flat_cols.numpy(),
            values=values32.numpy(), metadata=meta.numpy(), decoded=back.numpy(),
        )
        print(name, "ksp", int(ksp), "roundtrip", bool(torch.equal(back, t * mask_i.to(torch.float32))))


if __name__ == "__main__":
    main()
