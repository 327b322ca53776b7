"""End-to-end Python side: sparsifier, SrNMTensor, the Linear replacement."""
import numpy as np
import pytest
import torch

import oracle
from venom_amd.grouped_nmv_tensor import SrNMTensor, nm_vector_mask_sparsify


def test_sparsify_and_tensor_on_cpu():
    torch.manual_seed(0)
    rows, cols, n, m, v = 128, 96, 2, 8, 64
    w = torch.randn(rows, cols)
    masks, columns = nm_vector_mask_sparsify(w, n, m, v)
    omasks, ocols = oracle.select_columns(np.abs(w.numpy()), n, m, v)
    assert np.array_equal(masks.numpy(), omasks) and np.array_equal(columns.numpy(), ocols)
    t = SrNMTensor(n, m, v, w * masks, masks, columns, "cpu")
    assert t.values.dtype == torch.float16 and t.metadata.dtype == torch.int32 and t.columns.dtype == torch.int32
    assert (t.nrows, t.ncols, t.nnz) == (rows, cols, rows * 32)      # Ksp = ROUND_UP(12 * 2, 16) = 32
    ovals, ometa = oracle.encode((w * masks).numpy(), ocols.astype(np.uint32), n, m, v, mask=omasks)
    assert np.array_equal(t.values.numpy(), ovals.astype(np.float16))
    assert np.array_equal(t.metadata.numpy().view(np.uint32), ometa)
    assert torch.equal(t.to_dense(), (w * masks).half())


def test_fixed_pattern_sparsifier_shapes():
    from venom_amd.bert import NMVectorSparsifier

    w = torch.randn(128, 64)
    t = NMVectorSparsifier(2, 8, 64)(w).wrapped_tensor
    kept = torch.zeros(8)
    kept[0] = kept[2] = 1
    want = (w.reshape(128, 8, 8) * kept).reshape(128, 64).half()
    assert torch.equal(t.to_dense(), want)


@pytest.mark.gpu
def test_srnm_linear_matches_masked_dense_linear(gpu):
    from venom_amd.bert import SrnmSpmm

    torch.manual_seed(1)
    lin = torch.nn.Linear(256, 128).to(gpu).half()
    x = torch.randn(4, 24, 256, device=gpu).half()
    for magnitude in (False, True):
        sp = SrnmSpmm(lin, 2, 8, 64, magnitude=magnitude)
        y = sp(x)
        assert y.shape == (4, 24, 128)
        wd = SrNMTensor.to_dense(type("T", (), dict(values=sp.values, metadata=sp.metadata, columns=sp.columns, nrows=128,
                                                      ncols=256, n=2, m=8, tileM=64, device=gpu))())
        ref = x.float().reshape(-1, 256) @ wd.float().T
        ref = ref.half().float() + lin.bias.float()
        # relative to the entry unless it lies far below the result's typical magnitude (rms / 16)
        floor = ref.pow(2).mean().sqrt().item() / 16.0
        err = (y.float().reshape(-1, 128) - ref).abs() / ref.abs().clamp(min=floor)
        assert err.max().item() <= 1e-2


@pytest.mark.gpu
def test_bert_encoder_swap_runs_and_tracks_masked_dense(gpu):
    from venom_amd.bert import build_bert_large, linear_to_spmm, SrnmSpmm

    torch.set_grad_enabled(False)
    model = build_bert_large(layers=2).to(gpu).half()
    ids = torch.randint(0, 30522, (2, 64), device=gpu)
    sparse = linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64)
    swapped = [n for n, mod in sparse.named_modules() if isinstance(mod, SrnmSpmm)]
    assert len(swapped) == 2 * 6 and all("encoder.layer" in n for n in swapped)
    assert isinstance(sparse.pooler.dense, torch.nn.Linear)
    # a dense model whose encoder weights carry the same mask must give the same activations
    for name, mod in model.named_modules():
        if isinstance(mod, torch.nn.Linear) and "encoder.layer" in name:
            w = mod.weight
            kept = torch.zeros(8, device=gpu, dtype=w.dtype)
            kept[0] = kept[2] = 1
            mod.weight.copy_((w.reshape(w.shape[0], -1, 8) * kept).reshape(w.shape))
    a = sparse(ids).last_hidden_state.float()
    b = model(ids).last_hidden_state.float()
    assert torch.isfinite(a).all()
    assert (a - b).abs().max().item() <= 5e-2


def _mask_encoder_linears(model, gpu):
    """Gives the encoder Linears of a dense model the harness's fixed 2:8 pattern (entries 0 and 2 of every group)."""
    for name, mod in model.named_modules():
        if isinstance(mod, torch.nn.Linear) and "encoder.layer" in name:
            w = mod.weight
            kept = torch.zeros(8, device=gpu, dtype=w.dtype)
            kept[0] = kept[2] = 1
            mod.weight.copy_((w.reshape(w.shape[0], -1, 8) * kept).reshape(w.shape))
    return model


@pytest.mark.gpu
def test_bert_large_full_size_tracks_masked_dense(gpu):
    """The end-to-end configuration at full size: 24 layers, hidden 1024, 16 heads, feed-forward 4096, batch 32 x 512
    token ids over a 30522-entry vocabulary, every encoder Linear in 64:2:8 through the SpMM operator, against the dense
    fp16 model whose weights carry the same mask.  Both are fp16 evaluations of the same function; the tolerance is the
    one of the two-layer test, on every element of the last hidden state."""
    from venom_amd.bert import SrnmSpmm, build_bert_large, linear_to_spmm

    torch.set_grad_enabled(False)
    print("bert-large 24 layers, 32 x 512", flush=True)
    sparse = linear_to_spmm(build_bert_large(layers=24).to(gpu).half(), 2, 8, 64)
    assert sum(isinstance(mod, SrnmSpmm) for mod in sparse.modules()) == 24 * 6
    g = torch.Generator(device=gpu)
    g.manual_seed(0)
    ids = torch.randint(0, 30522, (32, 512), device=gpu, generator=g)
    a = sparse(ids).last_hidden_state.float()
    del sparse
    dense = _mask_encoder_linears(build_bert_large(layers=24).to(gpu).half(), gpu)
    b = dense(ids).last_hidden_state.float()
    assert a.shape == (32, 512, 1024) and torch.isfinite(a).all()
    diff = (a - b).abs()
    print("max abs difference %.4g, mean %.4g" % (diff.max().item(), diff.mean().item()), flush=True)
    assert diff.max().item() <= 5e-2


@pytest.mark.gpu
def test_gpt3_block_swap_tracks_masked_dense(gpu):
    """The GPT-3 block harness at reduced width (one GPT2Block, width 512, 8 heads, 1 x 256 tokens): its four Conv1D
    projections become SpMM layers over the transposed weight, and the block tracks the dense block whose weights carry
    the same mask.  128:2:16, the format of the GPT-3 feed-forward configuration."""
    from transformers.pytorch_utils import Conv1D
    from venom_amd.bert import SrnmSpmm
    from venom_amd.gpt2 import conv1d_to_spmm
    from venom_amd.gpt3 import build_gpt3_block

    torch.set_grad_enabled(False)
    width, heads, tokens, m = 512, 8, 256, 16
    dense = build_gpt3_block(width, heads, tokens).half().to(gpu)
    sparse = conv1d_to_spmm(build_gpt3_block(width, heads, tokens).half().to(gpu), 2, m, 128)
    assert sum(isinstance(mod, SrnmSpmm) for mod in sparse.modules()) == 4
    assert not any(isinstance(mod, Conv1D) for mod in sparse.modules())
    shapes = sorted((mod.nrows_sp, mod.ncols_sp) for mod in sparse.modules() if isinstance(mod, SrnmSpmm))
    assert shapes == sorted([(3 * width, width), (width, width), (4 * width, width), (width, 4 * width)])
    for mod in dense.modules():
        if isinstance(mod, Conv1D):
            w = mod.weight                                   # [in, out]
            kept = torch.zeros(m, device=gpu, dtype=w.dtype)
            kept[0] = kept[2] = 1
            wt = w.t().reshape(w.shape[1], -1, m) * kept
            mod.weight.copy_(wt.reshape(w.shape[1], w.shape[0]).t())
    x = torch.rand((1, tokens, width), device=gpu).half()
    a = sparse(x)
    b = dense(x)
    a = (a[0] if isinstance(a, tuple) else a).float()
    b = (b[0] if isinstance(b, tuple) else b).float()
    assert a.shape == (1, tokens, width) and torch.isfinite(a).all()
    assert (a - b).abs().max().item() <= 5e-2


def test_gpt3_harness_prints_the_reference_rows(capsys):
    """report_time of the GPT-3 harness: first field 2, then n, m (0, 0 for the dense row), V, mean, median, std, count
    (end2end/gpt3_pytorch.py:144-159)."""
    from venom_amd import gpt3

    gpt3.report_time("n:m", [0.002, 0.004], 2, 16, 128)
    gpt3.report_time("dense", [0.001], 2, 16, 128)
    rows = capsys.readouterr().out.strip().splitlines()
    f = rows[0].split(",")
    assert f[:4] == ["2", "2", "16", "128"] and abs(float(f[4]) - 3.0) < 1e-9 and f[-1] == "2"
    assert rows[1].split(",")[:4] == ["2", "0", "0", "128"]


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols", [(64, 64), (200, 328), (16384, 1024), (8, 4104), (37, 50)])
def test_transpose_matches_torch(gpu, rows, cols):
    from venom_amd import spatha
    x = torch.randn((rows, cols), device=gpu).half()
    assert torch.equal(spatha.transpose(x), x.T.contiguous())


@pytest.mark.gpu
def test_layer_reuses_transposed_input_only_for_the_same_activation(gpu):
    """Projections of one activation share its transposed copy; a changed or new activation never hits it."""
    from venom_amd import spatha
    from venom_amd.bert import SrnmSpmm

    torch.manual_seed(0)
    sp = [SrnmSpmm(torch.nn.Linear(128, 64).half().to(gpu), 2, 8, 64) for _ in range(2)]

    def direct(layer, x):       # the same product with the transposed copy made by torch
        rhs = x.reshape(-1, 128).T.contiguous()
        return spatha.spmm(layer.metadata, layer.columns, layer.values, rhs, layer.bias, 64, 128, rhs.shape[1], 64, 2, 8,
                           layer.nnz, 0, 32, 4).reshape(4, 32, 64)

    for trial in range(4):
        x = torch.randn((4, 32, 128), device=gpu).half()
        for layer in sp:
            assert torch.equal(layer(x), direct(layer, x))
        held = SrnmSpmm._last_rhs[2]
        sp[1](x)
        assert SrnmSpmm._last_rhs[2] is held            # second projection of the same activation: no new copy
        x.mul_(2)                                       # in-place change: the version counter moves
        assert torch.equal(sp[0](x), direct(sp[0], x))
        del x                                           # the next trial may or may not get the same address


@pytest.mark.gpu
def test_gpt2_conv1d_swap_tracks_masked_dense(gpu):
    """Every Conv1D of a small GPT-2 becomes an SpMM layer over the TRANSPOSED weight; a dense model whose
    weights carry the same mask gives the same activations."""
    from transformers.pytorch_utils import Conv1D
    from venom_amd.bert import SrnmSpmm
    from venom_amd.gpt2 import build_gpt2_large, conv1d_to_spmm

    torch.set_grad_enabled(False)
    dense = build_gpt2_large(layers=2, width=256, heads=4).to(gpu).half()
    sparse = conv1d_to_spmm(build_gpt2_large(layers=2, width=256, heads=4).to(gpu).half(), 2, 8, 64)
    swapped = [n for n, mod in sparse.named_modules() if isinstance(mod, SrnmSpmm)]
    assert len(swapped) == 2 * 4 and not any(isinstance(mod, Conv1D) for mod in sparse.modules())
    for mod in dense.modules():
        if isinstance(mod, Conv1D):
            w = mod.weight                                   # [in, out]; the mask runs along `in` for each output row
            kept = torch.zeros(8, device=gpu, dtype=w.dtype)
            kept[0] = kept[2] = 1
            wt = w.t().reshape(w.shape[1], -1, 8) * kept     # [out, in/8, 8]
            mod.weight.copy_(wt.reshape(w.shape[1], w.shape[0]).t())
    ids = torch.randint(0, 100, (2, 64), device=gpu)
    a = sparse(ids).last_hidden_state.float()
    b = dense(ids).last_hidden_state.float()
    assert torch.isfinite(a).all()
    assert (a - b).abs().max().item() <= 5e-2


@pytest.mark.gpu
def test_fused_feed_forward_tracks_the_unfused_layers(gpu):
    """BertIntermediate as one kernel (bias + GELU in the write-out, feature-major result consumed by the next
    layer without a copy) against the same model with the drop-in layers."""
    from venom_amd.bert import FusedFeedForwardIn, SrnmSpmm, build_bert_large, fuse_feed_forward, linear_to_spmm

    torch.set_grad_enabled(False)
    plain = linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64)
    fused = fuse_feed_forward(linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64))
    in_kernel = fuse_feed_forward(linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64), activation_in_kernel=True)
    assert sum(isinstance(mod, FusedFeedForwardIn) for mod in fused.modules()) == 2
    ids = torch.randint(0, 30522, (2, 64), device=gpu)
    a = plain(ids).last_hidden_state
    b = fused(ids).last_hidden_state
    c = in_kernel(ids).last_hidden_state.float()
    # bias in the kernel, torch's GELU on the feature-major buffer: the same numbers in another layout, bit for bit
    assert torch.equal(a, b)
    # GELU in the write-out as well: one fp16 step here and there
    assert torch.isfinite(c).all() and (a.float() - c).abs().max().item() <= 1e-2
    # the feature-major intermediate reaches the second feed-forward layer as a view: no transposed copy is made
    layer = fused.encoder.layer[0]
    x = torch.randn((2, 64, 1024), device=gpu).half()
    mid = layer.intermediate(x)
    assert mid.shape == (2, 64, 4096) and mid.stride() == (64, 1, 128)
    flat = torch.flatten(mid, 0, -2)
    assert SrnmSpmm._transposed(flat).data_ptr() == mid.data_ptr()
    want = torch.nn.functional.gelu(plain.encoder.layer[0].intermediate.dense(x))
    assert torch.equal(mid, want)


@pytest.mark.gpu
@pytest.mark.parametrize("in_kernel", [False, True])
def test_fused_gpt2_mlp_tracks_the_unfused_block(gpu, in_kernel):
    from venom_amd.bert import FusedFeedForwardIn, fuse_feed_forward
    from venom_amd.gpt2 import build_gpt2_large, conv1d_to_spmm

    torch.set_grad_enabled(False)
    plain = conv1d_to_spmm(build_gpt2_large(layers=2, width=256, heads=4).to(gpu).half(), 2, 8, 64)
    fused = fuse_feed_forward(conv1d_to_spmm(build_gpt2_large(layers=2, width=256, heads=4).to(gpu).half(), 2, 8, 64),
                              activation_in_kernel=in_kernel)
    assert sum(isinstance(mod, FusedFeedForwardIn) for mod in fused.modules()) == 2
    ids = torch.randint(0, 100, (2, 64), device=gpu)
    a = plain(ids).last_hidden_state
    b = fused(ids).last_hidden_state
    if in_kernel:      # one rounding instead of the eight of the block's elementwise chain
        assert (a.float() - b.float()).abs().max().item() <= 2e-2
    else:              # same operations on the same numbers in another layout
        assert torch.equal(a, b)


@pytest.mark.gpu
def test_merged_qkv_projection_gives_the_same_bits(gpu):
    from venom_amd.bert import build_bert_large, fuse_feed_forward, linear_to_spmm, merge_qkv

    torch.set_grad_enabled(False)
    plain = linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64)
    merged = merge_qkv(fuse_feed_forward(linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64)))
    for trial in range(2):          # a second input must not be served from the first one's result
        ids = torch.randint(0, 30522, (2, 64), device=gpu)
        assert torch.equal(plain(ids).last_hidden_state, merged(ids).last_hidden_state)
    att = merged.encoder.layer[0].attention.self
    x = torch.randn((2, 64, 1024), device=gpu).half()
    q, k, v = att.query(x), att.key(x), att.value(x)
    assert q.shape == (2, 64, 1024) and q.data_ptr() != k.data_ptr()
    for got, layer in ((q, plain.encoder.layer[0].attention.self.query), (k, plain.encoder.layer[0].attention.self.key),
                       (v, plain.encoder.layer[0].attention.self.value)):
        assert torch.equal(got, layer(x))


@pytest.mark.gpu
@pytest.mark.parametrize("tokens,hidden,with_residual", [(16384, 1024, True), (300, 1024, False), (64, 1280, True),
                                                          (7, 4096, True), (5, 8, True), (33, 72, False)])
def test_add_layernorm_matches_torch_addition_and_layer_norm(gpu, tokens, hidden, with_residual):
    """One kernel against the two it replaces.  The sum is rounded to fp16 in both; the statistics are accumulated in a
    different order (per-lane partial sums here, Welford there), so the fp32 results differ in the last bits and a few
    outputs land on the neighbouring fp16 value: at least 99 % equal, none more than one fp16 step apart
    (relative 2^-10) or, near zero, 1e-3 absolute."""
    from venom_amd import spatha

    g = torch.Generator(device=gpu)
    g.manual_seed(tokens * 31 + hidden)
    x = (torch.randn((tokens, hidden), generator=g, device=gpu) * 1.5 + 0.3).half()
    r = torch.randn((tokens, hidden), generator=g, device=gpu).half() if with_residual else None
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g, device=gpu)).half()
    b = (0.1 * torch.randn(hidden, generator=g, device=gpu)).half()
    got = spatha.add_layernorm(x, r, w, b, 1e-12)
    want = torch.nn.functional.layer_norm(x + r if with_residual else x, (hidden,), w, b, 1e-12)
    assert got.shape == want.shape and got.dtype == torch.float16
    assert (got == want).float().mean().item() >= 0.99
    diff = (got.float() - want.float()).abs()
    assert bool((diff <= torch.maximum(want.float().abs() * 2.0 ** -10, torch.tensor(1e-3, device=gpu))).all())
    # a 3-d activation is taken as [tokens, hidden] rows
    if tokens % 4 == 0:
        got3 = spatha.add_layernorm(x.view(4, tokens // 4, hidden), None if r is None else r.view(4, tokens // 4, hidden), w, b, 1e-12)
        assert torch.equal(got3.view(tokens, hidden), got)


@pytest.mark.gpu
@pytest.mark.parametrize("tokens,hidden,with_residual", [(16384, 1024, True), (304, 1024, False), (64, 1280, True), (40, 4096, True),
                                                          (8, 8, True), (72, 72, False), (1000, 512, True)])
def test_add_layernorm_feature_major_copy(gpu, tokens, hidden, with_residual):
    """The variant that writes its result twice: the row-major output equals the plain kernel's bit for bit, the second output is
    its transpose, and nothing is written outside either (guard bands)."""
    from venom_amd import _lib, spatha
    import ctypes

    print("layer norm, feature-major copy", tokens, hidden, with_residual, flush=True)
    g = torch.Generator(device=gpu)
    g.manual_seed(tokens * 31 + hidden)
    x = (torch.randn((tokens, hidden), generator=g, device=gpu) * 1.5 + 0.3).half()
    r = torch.randn((tokens, hidden), generator=g, device=gpu).half() if with_residual else None
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g, device=gpu)).half()
    b = (0.1 * torch.randn(hidden, generator=g, device=gpu)).half()
    want = spatha.add_layernorm(x, r, w, b, 1e-12)
    out, out_t = spatha.add_layernorm(x, r, w, b, 1e-12, feature_major=True)
    assert tuple(out_t.shape) == (hidden, tokens) and out_t.is_contiguous()
    assert torch.equal(out, want) and torch.equal(out_t, want.t())
    # through the C ABI into buffers with guard bands
    guard = 2048
    n = tokens * hidden
    buf = torch.full((2 * n + 3 * guard,), 7.0, dtype=torch.float16, device=gpu)
    o1, o2 = buf[guard:guard + n], buf[2 * guard + n:2 * guard + 2 * n]
    stream = ctypes.c_void_p(torch.cuda.current_stream(gpu).cuda_stream)
    _lib.check(_lib.lib().spatha_add_layernorm_f16_t(x.data_ptr(), None if r is None else r.data_ptr(), w.data_ptr(), b.data_ptr(), 1e-12,
                                                     tokens, hidden, o1.data_ptr(), o2.data_ptr(), stream), "ln_t")
    torch.cuda.synchronize()
    assert torch.equal(o1.view(tokens, hidden), want) and torch.equal(o2.view(hidden, tokens), want.t())
    assert bool((buf[:guard] == 7.0).all()) and bool((buf[guard + n:2 * guard + n] == 7.0).all()) and bool((buf[2 * guard + 2 * n:] == 7.0).all())
    if tokens == 8:
        with pytest.raises(_lib.SpathaError):           # tokens % 8
            spatha.add_layernorm(x[:5].contiguous(), None, w, b, 1e-12, feature_major=True)


@pytest.mark.gpu
def test_feature_major_layer_norm_feeds_the_next_projection(gpu):
    """The encoder with the residual + LayerNorm kernel handing its feature-major copy to the next SrnmSpmm: same output as with the
    plain fused kernel (the projections read the same numbers, only who transposes them changes), and the library's transpose kernel
    runs once per layer instead of three times."""
    from venom_amd import spatha
    from venom_amd.bert import build_bert_large, fuse_add_layernorm, linear_to_spmm

    torch.set_grad_enabled(False)
    torch.manual_seed(3)
    plain = fuse_add_layernorm(linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64))
    torch.manual_seed(3)
    handed = fuse_add_layernorm(linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64), feature_major=True)
    ids = torch.randint(0, 30522, (2, 64), device=gpu)
    calls = []
    real = spatha.transpose
    try:
        spatha.transpose = lambda t: (calls.append(tuple(t.shape)), real(t))[1]
        a = plain(ids).last_hidden_state
        n_plain = len(calls)
        calls.clear()
        b = handed(ids).last_hidden_state
        n_handed = len(calls)
    finally:
        spatha.transpose = real
    assert torch.equal(a, b)
    # per layer: q/k/v input, attention context, FFN-up input, FFN-down input -> the first layer keeps all but one (its q/k/v input
    # comes from the embeddings), every later layer keeps the context and the FFN-down input only
    assert n_plain == 8 and n_handed == 5, (n_plain, n_handed)


@pytest.mark.gpu
def test_add_layernorm_rejects_what_the_kernel_does_not_take(gpu):
    from venom_amd import _lib, spatha

    x = torch.zeros((4, 12), device=gpu).half()           # hidden not a multiple of 8
    w = torch.ones(12, device=gpu).half()
    with pytest.raises(_lib.SpathaError):
        spatha.add_layernorm(x, None, w, w, 1e-5)
    x = torch.zeros((2, 8192), device=gpu).half()         # more than a lane's registers hold
    w = torch.ones(8192, device=gpu).half()
    with pytest.raises(_lib.SpathaError):
        spatha.add_layernorm(x, None, w, w, 1e-5)
    with pytest.raises(ValueError):
        spatha.add_layernorm(torch.zeros((2, 16), device=gpu).half(), torch.zeros((2, 8), device=gpu).half(),
                             torch.ones(16, device=gpu).half(), torch.ones(16, device=gpu).half(), 1e-5)


@pytest.mark.gpu
def test_fused_projection_norm_tracks_the_stock_modules(gpu):
    from venom_amd.bert import FusedProjectionNorm, build_bert_large, fuse_add_layernorm, linear_to_spmm

    torch.set_grad_enabled(False)
    torch.manual_seed(3)
    stock = linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64)
    torch.manual_seed(3)
    fused = fuse_add_layernorm(linear_to_spmm(build_bert_large(layers=2).to(gpu).half(), 2, 8, 64))
    assert isinstance(fused.encoder.layer[0].output, FusedProjectionNorm)
    assert isinstance(fused.encoder.layer[1].attention.output, FusedProjectionNorm)
    ids = torch.randint(0, 30522, (2, 64), device=gpu)
    a, b = stock(ids).last_hidden_state.float(), fused(ids).last_hidden_state.float()
    assert (a - b).abs().max().item() <= 2e-2 and ((a - b).abs() <= 2e-3).float().mean().item() >= 0.99
    fused.train()                                            # in training the stock sequence runs (dropout is live)
    assert fused.encoder.layer[0].output(torch.zeros((1, 8, 4096), device=gpu).half(),
                                         torch.zeros((1, 8, 1024), device=gpu).half()).shape == (1, 8, 1024)
