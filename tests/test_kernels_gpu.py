"""Each HIP kernel alone against its plain reference (tests/reference_ops.py), at sizes other than
the engine's tiny models: odd row counts, widths and vocabularies that are no power of two,
scattered pages, contexts at page edges."""
import math

import numpy as np
import pytest
import torch

import plain_llama
from reference_ops import ReferenceOps

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from fllm_amd.kernels import Ops
    return Ops(library_gemm_from=None)      # the hand-written kernels at every size


@pytest.fixture(scope="module")
def library_ops():
    from fllm_amd.kernels import Ops
    return Ops(library_gemm_from=17)        # bfloat16 products of 17 rows and more through the GEMM library


@pytest.fixture(scope="module")
def ref():
    return ReferenceOps()


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def close(got, want, rtol, atol, what=""):
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    worst = (err - bound).max().item()
    assert worst <= 0, f"{what}: max err {err.max().item():.3e} (|want| max {want.abs().max().item():.3e}), over bound by {worst:.3e}"


BF16_EPS = 2.0 ** -8


# ---------------------------------------------------------------------------------------------
# random weights: the device draws what the host draws
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1,), (5,), (130, 77), ((1 << 21) + 3,), (515, 4099)])
def test_random_weights_are_the_same_bits_on_the_host_and_on_the_device(ops, dtype, shape):
    from fllm_amd.parts.base import INIT_MATRIX, INIT_NORM
    from fllm_amd.weights.random_init import random_tensor
    as_int = torch.int32 if dtype == torch.float32 else torch.int16
    for kind in (INIT_MATRIX, INIT_NORM):
        host = random_tensor("model.layers.3.x.weight", shape, kind, 12, dtype, "cpu")
        device = random_tensor("model.layers.3.x.weight", shape, kind, 12, dtype, DEV, ops)
        assert device.is_cuda and device.shape == host.shape and device.dtype == dtype
        differ = (host.view(as_int) != device.cpu().view(as_int)).sum().item()
        assert differ == 0, f"{kind} {dtype} {shape}: {differ} elements differ"


def test_random_model_on_the_device_is_the_model_of_the_host():
    """An engine whose random weights are drawn on the device computes what the plain implementation computes from the
    weights drawn on the host: a benchmark's model can be replayed."""
    import tiny_configs as tc
    from fllm_amd import Engine, SamplingParams
    from fllm_amd.registry import model_spec_from_config
    from fllm_amd.weights import random_tensors
    cfg = tc.TINY_A
    _, spec = model_spec_from_config(cfg)
    host = random_tensors(spec, 4, torch.float32)
    on_device = random_tensors(spec, 4, torch.float32, device=DEV)
    assert all(torch.equal(host[n], on_device[n].cpu()) for n in host)
    engine = Engine(config=cfg, seed=4, dtype="float32", ctx=128, max_seqs=2, block_size=16, num_blocks=16,
                    random_weights_on_device=True)
    prompt = tc.random_ids(9, cfg["vocab_size"], 3)
    tokens = engine.generate([prompt], SamplingParams(max_tokens=6))[0]
    w64, seq = tc.to_float64(host), list(prompt)
    for t in tokens:
        assert t == plain_llama.greedy(plain_llama.forward(cfg, w64, seq)[-1])
        seq.append(t)


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,vocab", [(1, 64, 256), (13, 160, 515), (5, 4104, 1000)])
def test_embed(ops, ref, dtype, rows, width, vocab):
    g = gen(1)
    table = torch.randn(vocab, width, generator=g).to(dtype)
    ids = torch.randint(0, vocab, (rows,), generator=g, dtype=torch.int32)
    ids[0] = vocab - 1
    want = ref.embed(ids, table, torch.empty(rows, width), 1.0)
    got = ops.embed(ids.to(DEV), table.to(DEV), torch.empty(rows, width, device=DEV), 1.0)
    assert torch.equal(got.cpu(), want)
    got = ops.embed(ids.to(DEV), table.to(DEV), torch.empty(rows, width, device=DEV), 0.5)
    assert torch.equal(got.cpu(), want * 0.5)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,eps", [(1, 64, 1e-5), (13, 160, 1e-6), (5, 4096, 1e-5), (3, 5144, 1e-3)])
def test_rmsnorm(ops, ref, out_dtype, rows, width, eps):
    g = gen(2)
    x = torch.randn(rows, width, generator=g) * 3.0
    w = 1.0 + 0.1 * torch.randn(width, generator=g)
    want = ref.rmsnorm(x, w, eps, torch.empty(rows, width, dtype=torch.float64))
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, torch.empty(rows, width, dtype=out_dtype, device=DEV))
    tol = 2e-6 if out_dtype == torch.float32 else BF16_EPS
    close(got, want, tol, tol * 1e-3, "rmsnorm")
    # row selection, in an order of its own
    sel = torch.tensor([rows - 1, 0, rows - 1], dtype=torch.int32)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, torch.empty(3, width, dtype=out_dtype, device=DEV), rows=sel.to(DEV))
    close(got, want[sel.long()], tol, tol * 1e-3, "rmsnorm rows")


@pytest.mark.parametrize("branch_dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("rows,width", [(1, 64), (13, 4096), (5, 5140), (3, 8192), (2, 9000), (4, 1001)])
def test_add_rmsnorm(ops, ref, branch_dtype, out_dtype, rows, width):
    g = gen(41)
    x = torch.randn(rows, width, generator=g) * 2
    branch = torch.randn(rows, width, generator=g).to(branch_dtype)
    w = 1.0 + 0.1 * torch.randn(width, generator=g)
    x_ref = x.double()
    want = ref.add_rmsnorm(x_ref, branch, w, 1e-5, torch.empty(rows, width, dtype=torch.float64))
    x_gpu = x.to(DEV)
    got = ops.add_rmsnorm(x_gpu, branch.to(DEV), w.to(DEV), 1e-5, torch.empty(rows, width, dtype=out_dtype, device=DEV))
    assert torch.equal(x_gpu.cpu(), x + branch.float())
    tol = 2e-6 if out_dtype == torch.float32 else BF16_EPS
    close(got, want, tol, tol * 1e-3, "add_rmsnorm")


def test_rmsnorm_row_is_the_same_alone_and_in_a_batch(ops):
    g = gen(3)
    x = torch.randn(9, 1000, generator=g).to(DEV)
    w = torch.randn(1000, generator=g).to(DEV)
    full = ops.rmsnorm(x, w, 1e-5, torch.empty(9, 1000, device=DEV))
    one = ops.rmsnorm(x[4:5].contiguous(), w, 1e-5, torch.empty(1, 1000, device=DEV))
    assert torch.equal(full[4:5], one)


def _linear_case(ops, ref, dtype, M, N, K, mode, bias, seed=4, branch_rounded=False):
    g = gen(seed)
    x = (torch.randn(M, K, generator=g)).to(dtype)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    b = torch.randn(N, generator=g) if bias else None
    if mode == "store":
        out_dtype = dtype
    else:
        out_dtype = torch.float32
    base = torch.randn(M, N, generator=g) if mode == "add" else torch.zeros(M, N)
    want = base.double().clone()
    ref.linear(x, w, want, bias=b, accumulate=True)
    out = base.to(out_dtype).to(DEV)
    ops.linear(x.to(DEV), w.to(DEV), out, bias=None if b is None else b.to(DEV), accumulate=(mode == "add"))
    # float32 accumulation of K products of magnitude ~|x||w|: a few units of 2^-24 * sqrt(K) * magnitude
    mag = (x.double().abs() @ w.double().abs().T).max().item()
    atol = 4e-7 * mag + 1e-6
    rtol = BF16_EPS if out_dtype == torch.bfloat16 else 1e-6
    if branch_rounded:      # the library product is rounded to bfloat16 before it is added
        atol += BF16_EPS * (want - base.double()).abs().max().item()
    close(out, want, rtol, atol + (BF16_EPS * 1e-2 if out_dtype == torch.bfloat16 else 0), f"linear {dtype} M{M} N{N} K{K} {mode}")


@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 176, 64), (13, 100, 72), (70, 130, 200), (2, 515, 33)])
@pytest.mark.parametrize("mode,bias", [("store", False), ("f32", True), ("add", True)])
def test_linear_f32(ops, ref, M, N, K, mode, bias):
    _linear_case(ops, ref, torch.float32, M, N, K, mode, bias)


def test_linear_f32_row_is_the_same_alone_and_in_a_batch(ops):
    g = gen(5)
    x = torch.randn(77, 300, generator=g).to(DEV)
    w = torch.randn(130, 300, generator=g).to(DEV)
    full = ops.linear(x, w, torch.empty(77, 130, device=DEV))
    one = ops.linear(x[70:71].contiguous(), w, torch.empty(1, 130, device=DEV))
    assert torch.equal(full[70:71], one)


SKINNY = [(1, 16, 64), (1, 4096, 4096), (2, 100, 136), (5, 6144, 4096), (8, 4096, 14336), (16, 520, 264),
          (17, 128, 128), (33, 1000, 4096), (64, 4096, 4096), (48, 30, 72),
          # 8-row weight tiles with two K halves (up to 8 rows, 4,100 to 16,000 outputs), ragged in N and K
          (3, 5001, 64), (7, 6148, 200), (8, 4104, 1096), (1, 9000, 520),
          # 17 to 64 rows: a K slice of the activations stays in LDS, a workgroup a compute unit, K slices over workgroups
          (20, 4096, 14336), (64, 6144, 4096), (40, 100, 264), (33, 5001, 72), (64, 48, 8192), (18, 28672, 512),
          (64, 4096, 14336), (64, 28672, 4096), (64, 4096, 8192), (64, 8200, 1000), (17, 16, 24), (50, 1000, 2072),
          # K in slices over workgroups (the rows of all of K do not fit into LDS), 8 and 16 waves
          (16, 136, 14336), (5, 1000, 30008), (12, 72, 65536)]
TILED = [(65, 128, 64), (128, 200, 200), (200, 6144, 4096), (300, 130, 136), (2048, 512, 4096), (129, 4096, 14336)]
PLAIN = [(3, 50, 100), (70, 64, 36)]      # K not a multiple of 8: the plain kernel


@pytest.mark.parametrize("M,N,K", SKINNY + TILED + PLAIN)
@pytest.mark.parametrize("mode,bias", [("store", False), ("f32", True), ("add", True)])
def test_linear_bf16(ops, ref, M, N, K, mode, bias):
    _linear_case(ops, ref, torch.bfloat16, M, N, K, mode, bias)


@pytest.mark.parametrize("M,N,K", [(17, 128, 128), (64, 4096, 4096), (200, 6144, 4096), (300, 130, 136)])
@pytest.mark.parametrize("mode,bias", [("store", False), ("add", False), ("f32", False), ("add", True)])
def test_linear_bf16_library_path(library_ops, ref, M, N, K, mode, bias):
    _linear_case(library_ops, ref, torch.bfloat16, M, N, K, mode, bias, branch_rounded=(mode == "add" and not bias))


@pytest.mark.parametrize("K,row_counts", [(4096, (1, 8, 16, 64)), (2048, (1,)), (8192, (1,))])
def test_vocabulary_projection_at_the_benchmark_sizes(ops, library_ops, K, row_counts):
    """The product that ends every step, at the sizes the benchmark times: 128,256 outputs in float32 from bfloat16
    operands, widths of the 8B, 1B and 70B shapes; up to 16 rows on this library's kernel, 64 rows through the GEMM
    library as the engine sends them.  Against the float64 product.  On this library's kernel a row's bits do not depend
    on the rows beside it; up to 8 rows (one tile shape) they are also the bits of the row computed alone."""
    N = 128256
    g = gen(46)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    x = torch.randn(max(row_counts), K, generator=g).to(torch.bfloat16)
    w64, wg = w.double(), w.to(DEV)
    want = x.double() @ w64.T
    mag = (x.double().abs() @ w64.abs().T).max().item()
    alone = None
    for M in row_counts:
        which = library_ops if M > 16 else ops
        out = which.linear(x[:M].to(DEV), wg, torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV))
        close(out, want[:M], 1e-6, 4e-7 * mag + 1e-6, f"vocabulary projection M{M} K{K}")
        assert torch.equal(out.argmax(-1).cpu(), want[:M].argmax(-1)), f"M{M} K{K}: another largest logit"
        if M == 1:
            alone = out[0].clone()
        elif M <= 16:
            if M <= 8:
                assert torch.equal(out[0], alone), f"M{M} K{K}: row 0 differs from the row computed alone"
            others = x[:M].clone()
            others[1:] = torch.randn(M - 1, K, generator=g).to(torch.bfloat16)
            again = which.linear(others.to(DEV), wg, torch.empty((M, N), dtype=torch.float32, device=DEV))
            assert torch.equal(again[0], out[0]), f"M{M} K{K}: row 0 depends on the rows beside it"


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 4096, 14336), (16, 2048, 8192), (5, 4104, 1024), (8, 40, 1024), (3, 8192, 2048),
                                   (16, 4096, 14336), (2, 24, 3072), (9, 1000, 2048)])
@pytest.mark.parametrize("bias", [False, True])
def test_products_that_add_read_the_tile_major_copy(ops, ref, M, N, K, bias):
    """The output and down projections of decode steps keep a second copy of their matrix, tile by tile in the order the
    lanes of a wave take it (`Ops.tile_for_decode`): `linear(..., accumulate=True)` and `linear_add_prepare` find it by
    the matrix's address.  The sums are those of the row-major matrix bit for bit (the same products in the same order),
    and the float64 product's within rounding; the copy holds every element at its place."""
    g = gen(47)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    b = torch.randn(N, generator=g).to(DEV) if bias else None
    base = torch.randn(M, N, generator=g).to(DEV)
    plain = ops.linear(x, w, base.clone(), bias=b, accumulate=True)
    twin = w.clone()                                         # the same values at another address: that one gets the copy
    assert ops.tile_for_decode(twin) and ops._tiles_of(twin) is not None and ops._tiles_of(w) is None
    tiles = ops._tiles_of(twin).view(-1, K // 128, 4, 4, 16, 8)          # [tile][block][k-step][lane / 16][lane % 16][8]
    back = tiles.permute(0, 4, 1, 2, 3, 5).reshape(-1, K)                 # [16 tile + lane % 16][128 block + 32 step + 8 (lane / 16) + j]
    assert torch.equal(back[:N], w) and not back[N:].any()
    tiled = ops.linear(x, twin, base.clone(), bias=b, accumulate=True)
    assert torch.equal(tiled, plain), f"M{M} N{N} K{K}: the tile-major copy gives other sums"
    want = ref.linear(x.cpu(), w.cpu(), base.double().cpu(), bias=None if b is None else b.cpu(), accumulate=True)
    mag = (x.double().abs() @ w.double().abs().T).max().item()
    close(tiled, want, 1e-6, 4e-7 * mag + 1e-6, f"tile-major M{M} N{N} K{K}")
    if N % 16 == 0:
        norm_w = (1.0 + 0.1 * torch.randn(N, generator=g)).to(DEV)
        r1, r2 = base.clone(), base.clone()
        a = ops.linear_add_prepare(x, w, r1, norm_w, bias=b)
        c = ops.linear_add_prepare(x, twin, r2, norm_w, bias=b)
        assert torch.equal(r1, r2) and torch.equal(a.x, c.x) and a.parts == c.parts
        assert torch.equal(a.ssq[:M * a.parts], c.ssq[:M * c.parts])
    key = twin.data_ptr()
    del twin, tiles, back
    assert key not in type(ops)._tiles                       # the copy goes with its matrix
    assert not ops.tile_for_decode(torch.zeros(64, 1000, dtype=torch.bfloat16, device=DEV))       # widths it does not take
    assert not ops.tile_for_decode(torch.zeros(64, 1024, dtype=torch.float32, device=DEV))


@pytest.mark.parametrize("M,N,K,bias", [(1, 128256, 4096, False), (8, 128256, 2048, False), (16, 32000, 1024, True), (3, 1000, 2048, True),
                                        (5, 50280, 3072, False), (16, 4104, 8192, False), (17, 1000, 2048, False), (33, 32000, 1024, True),
                                        (64, 128256, 2048, False), (48, 50280, 4096, False)])
def test_the_vocabulary_projection_reads_the_tile_major_copy(ops, ref, M, N, K, bias):
    """float32 logits of up to 64 rows from the tile-major copy of the matrix, where there is one: the float64 product's
    within rounding, and a row alone what it is in the batch where the launch has the same form."""
    g = gen(53 + M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    b = torch.randn(N, generator=g).to(DEV) if bias else None
    plain = ops.linear(x, w, torch.empty(M, N, device=DEV), bias=b)
    assert ops.tile_for_decode(w)
    tiled = ops.linear(x, w, torch.empty(M, N, device=DEV), bias=b)
    want = ref.linear(x.cpu(), w.cpu(), torch.empty(M, N, dtype=torch.float64), bias=None if b is None else b.cpu())
    mag = (x.double().abs() @ w.double().abs().T).max().item()
    close(tiled, want, 1e-6, 4e-7 * mag + 1e-6, f"logits from the tile-major copy M{M} N{N} K{K}")
    close(tiled, plain.double().cpu(), 1e-6, 4e-7 * mag + 1e-6, f"logits, copy against matrix M{M} N{N} K{K}")
    if M <= 16 and N >= 32000:          # launches of the same form whatever the rows: the same sums in the same order
        alone = ops.linear(x[:1], w, torch.empty(1, N, device=DEV), bias=b)
        assert torch.equal(alone[0], tiled[0]), "row 0 depends on the rows beside it"


@pytest.mark.parametrize("waves", [0, 4, 7, 8])
@pytest.mark.parametrize("M,N,K,bias", [(17, 4096, 4096, False), (64, 4096, 14336, False), (33, 1000, 2048, True), (48, 24, 1024, True),
                                        (64, 4104, 3072, False), (20, 16, 7168, False)])
def test_products_of_17_to_64_rows_that_add_read_the_tile_major_copy(ops, ref, M, N, K, bias, waves):
    """From 17 rows on the products that add into the residual stream take four to eight row tiles a workgroup and the
    activations through LDS in chunks; with the tile-major copy they read 1 KiB a load instruction and may take
    workgroups of seven or eight waves (`linear.wide_waves`; 0 lets the plan choose).  The sums are those of the row-major
    matrix bit for bit whatever the number of waves, and the float64 product's within rounding."""
    g = gen(53)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    b = torch.randn(N, generator=g).to(DEV) if bias else None
    base = torch.randn(M, N, generator=g).to(DEV)
    from fllm_amd.kernels import _ptr
    plain = base.clone()                                     # the row-major matrix through the same kernel
    ops._check(ops.lib.fllm_linear_add_tiled(_ptr(x), x.stride(0), _ptr(w), None, _ptr(b), _ptr(plain), N, M, N, K, ops._stream()))
    twin = w.clone()
    assert ops.tile_for_decode(twin)
    ops.set_option("linear.wide_waves", waves)
    try:
        tiled = ops.linear(x, twin, base.clone(), bias=b, accumulate=True)
        again = ops.linear(x, twin, base.clone(), bias=b, accumulate=True)
    finally:
        ops.set_option("linear.wide_waves", 0)
    assert torch.equal(tiled, again), "two launches differ"
    want = ref.linear(x.cpu(), w.cpu(), base.double().cpu(), bias=None if b is None else b.cpu(), accumulate=True)
    mag = (x.double().abs() @ w.double().abs().T).max().item()
    close(tiled, want, 1e-6, 4e-7 * mag + 1e-6, f"tile-major M{M} N{N} K{K} waves {waves}")
    # the slices a plan cuts K into depend on the number of waves, and with them the order of the sums: bit-equal to the
    # row-major matrix under the plan that the row-major matrix gets (four waves)
    ops.set_option("linear.wide_waves", 4)
    try:
        four = ops.linear(x, twin, base.clone(), bias=b, accumulate=True)
    finally:
        ops.set_option("linear.wide_waves", 0)
    assert torch.equal(four, plain), f"M{M} N{N} K{K}: the tile-major copy gives other sums"


@pytest.mark.parametrize("M,N,K,bias", [(65, 4096, 4096, False), (128, 4096, 14336, False), (96, 1000, 2048, True), (100, 24, 1024, True),
                                        (128, 4104, 3072, False), (97, 2048, 8192, False), (80, 16, 7168, True), (72, 4096, 14336, False),
                                        (112, 2048, 4096, False)])
def test_products_of_65_to_128_rows(ops, ref, M, N, K, bias):
    """65 to 128 rows: five to eight row tiles a workgroup of eight waves, from the tile-major copies only, for the two
    products of the feed-forward.  The sum into the residual stream with and without the preparation of the next norm and
    gate/up from bfloat16 rows, each against the float64 result; two launches give the same bits; the other forms refuse."""
    g = gen(61 + M)
    x = (torch.randn(M, K, generator=g) * 0.5).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    b = (torch.randn(N, generator=g) * 0.1).to(DEV) if bias else None
    resid = (torch.randn(M, N, generator=g) * torch.rand(M, 1, generator=g) * 6).to(DEV)
    assert ops.tile_for_decode(w)
    want = ref.linear(x.cpu(), w.cpu(), resid.double().cpu(), bias=None if b is None else b.cpu(), accumulate=True)
    mag = (x.double().abs() @ w.double().abs().T).max().item()
    summed = ops.linear(x, w, resid.clone(), bias=b, accumulate=True)
    close(summed, want, 1e-6, 4e-7 * mag + 1e-6, f"sum M{M} N{N} K{K}")
    assert torch.equal(summed, ops.linear(x, w, resid.clone(), bias=b, accumulate=True)), "two launches differ"
    with pytest.raises(Exception, match="tile-major copy|steps of 256"):
        ops.gate_up_swiglu(x, torch.zeros(64, K, dtype=torch.bfloat16, device=DEV), torch.empty(M, 32, dtype=torch.bfloat16, device=DEV))
    if N % 1024 != 0:
        return
    nw = (1 + 0.1 * torch.randn(N, generator=g)).to(DEV)
    assert ops.fused_form(M, K, w) is None and not ops.prepares_norm(M, N, w)      # steps of this many rows do not use it
    prepared_sum = resid.clone()
    prepared = ops.linear_add_prepare(x, w, prepared_sum, nw, bias=b)
    assert torch.equal(prepared_sum, summed)
    assert torch.equal(prepared.x, (summed * nw).to(torch.bfloat16)) and prepared.parts == N // 16
    squares = prepared.ssq[:M * prepared.parts].view(M, prepared.parts).double().sum(1)
    assert float(((squares - summed.double().pow(2).sum(1)).abs() / summed.double().pow(2).sum(1)).max()) < 1e-6
    inter = 3 * N // 2 + 8
    wgu = (torch.randn(2 * inter, N, generator=g) / math.sqrt(N)).to(torch.bfloat16).to(DEV)
    bgu = (torch.randn(2 * inter, generator=g) * 0.1).to(DEV)
    assert ops.tile_for_decode(wgu, gate_up=True)
    want_act = ref.norm_gate_up_swiglu(summed.cpu(), nw.cpu(), 1e-5, wgu.cpu(), torch.empty(M, inter, dtype=torch.float64), bias=bgu.cpu())
    normed = ops.rmsnorm(summed, nw, 1e-5, torch.empty(M, N, dtype=torch.bfloat16, device=DEV))
    act = ops.gate_up_swiglu(normed, wgu, torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), bias=bgu)
    close(act, want_act, 2 * BF16_EPS, 4e-2, f"gate/up M{M} N{N}")
    assert torch.equal(act, ops.gate_up_swiglu(normed, wgu, torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), bias=bgu))
    with pytest.raises(Exception, match="1..64 rows"):
        ops.norm_gate_up_swiglu(None, None, 1e-5, wgu, torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), bias=bgu, prepared=prepared)


@pytest.mark.parametrize("waves", [0, 4, 7, 8])
@pytest.mark.parametrize("M,inter,K,bias", [(17, 14336, 4096, False), (64, 14336, 4096, False), (40, 1000, 2048, True), (64, 12, 1024, True),
                                            (29, 8192, 2048, False), (64, 1796, 1024, False)])
def test_gate_up_of_17_to_64_rows_reads_the_tile_major_copy(ops, ref, M, inter, K, bias, waves):
    """`gate_up_swiglu` from 17 rows on with the copy that holds 8 gate rows and the same 8 up rows a tile
    (`tile_for_decode(w, gate_up=True)`): the copy holds every element at its place, the outputs are those of the
    row-major matrix bit for bit (one slice of K: the same products in the same order) and the float64 result's within
    bfloat16 rounding."""
    g = gen(59)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(2 * inter, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    b = torch.randn(2 * inter, generator=g).to(DEV) if bias else None
    from fllm_amd.kernels import _ptr
    plain = torch.empty((M, inter), dtype=torch.bfloat16, device=DEV)        # the row-major matrix through the same kernel
    ops._check(ops.lib.fllm_gate_up_swiglu_tiled(_ptr(x), x.stride(0), _ptr(w), None, _ptr(b), _ptr(plain), M, inter, K, ops._stream()))
    twin = w.clone()
    assert ops.tile_for_decode(twin, gate_up=True) and ops._tiles_of(twin) is None and ops._tiles_of(twin, gate_up=True) is not None
    tiles = ops._tiles_of(twin, gate_up=True).view(-1, K // 128, 4, 4, 2, 8, 8)     # [tile][block][k-step][lane / 16][gate, up][row % 8][8]
    back = tiles.permute(4, 0, 5, 1, 2, 3, 6).reshape(2, -1, K)                      # [gate, up][8 tile + row % 8][128 block + 32 step + 8 (lane / 16) + j]
    assert torch.equal(back[0, :inter], w[:inter]) and torch.equal(back[1, :inter], w[inter:]) and not back[:, inter:].any()
    ops.set_option("linear.wide_waves", waves)
    try:
        tiled = ops.gate_up_swiglu(x, twin, torch.empty((M, inter), dtype=torch.bfloat16, device=DEV), bias=b)
    finally:
        ops.set_option("linear.wide_waves", 0)
    want = ref.gate_up_swiglu(x.cpu(), w.cpu(), torch.empty((M, inter), dtype=torch.float64), bias=None if b is None else b.cpu())
    close(tiled.float(), want, 2 * BF16_EPS, 1e-4, f"gate/up tile-major M{M} I{inter} K{K} waves {waves}")
    same = (tiled == plain).float().mean().item()        # another number of waves may cut K into other slices
    assert same == 1.0 if waves == 4 else same > 0.999, f"M{M} I{inter} K{K} waves {waves}: {1 - same:.2%} of the outputs differ from the row-major matrix's"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 64), (13, 4099), (300, 4096)])
def test_add_residual(ops, dtype, rows, width):
    g = gen(40)
    residual = torch.randn(rows, width, generator=g)
    branch = torch.randn(rows, width, generator=g).to(dtype)
    got = ops.add_residual(residual.to(DEV), branch.to(DEV))
    assert torch.equal(got.cpu(), residual + branch.float())


@pytest.mark.parametrize("M,N,K,option,values", [
    (8, 6144, 4096, "linear.dual_k", (0, 1)), (3, 5001, 200, "linear.dual_k", (0, 1)),
    (8, 4096, 14336, "linear.x_direct", (0, 1)), (16, 1000, 520, "linear.x_direct", (0, 1)), (3, 5001, 200, "linear.x_direct", (0, 1)),
    (8, 4096, 14336, "linear.slices", (0, 2, 4, 8)), (2, 1000, 4096, "linear.slices", (0, 2, 4)),
    (16, 264, 8192, "linear.slices", (0, 4)), (64, 4096, 14336, "linear.slices", (0, 1, 2, 4, 8, 14, 19)), (40, 1000, 4096, "linear.slices", (0, 1, 2, 4, 6)),
    (64, 4096, 14336, "linear.slab", (0, 1, 2)), (33, 5001, 72, "linear.slab", (0, 2)), (48, 6144, 4096, "linear.slab", (0, 2)),
    (64, 28672, 4096, "linear.slab", (0, 2)), (20, 128256, 1024, "linear.slab", (0, 2))])
def test_linear_bf16_variants_agree(ops, ref, M, N, K, option, values):
    """The ways of cutting a decode-shaped product (tile shape, K slices) give the same sums up to the order
    of float32 additions, each of them the same bits on every call."""
    g = gen(44)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    want = ref.linear(x, w, torch.zeros(M, N, dtype=torch.float64))
    mag = (x.double().abs() @ w.double().abs().T).max().item()
    xg, wg = x.to(DEV), w.to(DEV)
    try:
        if option == "linear.slices":
            ops.set_option("linear.x_direct", 0)      # slices exist for staged activations only
        for value in values:
            ops.set_option(option, value)
            outs = [ops.linear(xg, wg, torch.empty(M, N, dtype=torch.float32, device=DEV)) for _ in range(4)]
            close(outs[0], want, 1e-6, 4e-7 * mag + 1e-6, f"{option}={value}")
            for other in outs[1:]:
                assert torch.equal(other, outs[0]), f"{option}={value}: two calls differ"
    finally:
        ops.set_option(option, 0 if option == "linear.slices" else 1)
        ops.set_option("linear.x_direct", 1)


def test_sliced_products_leave_their_counters_at_zero(ops, ref):
    """Products of different shapes share the counters of the K-sliced form: each must hand them back at zero."""
    g = gen(45)
    ops.set_option("linear.x_direct", 0)
    try:
        _sliced_products(ops, ref, g)
    finally:
        ops.set_option("linear.x_direct", 1)


def _sliced_products(ops, ref, g):
    for M, N, K in [(8, 4096, 14336), (5, 1000, 30008), (16, 136, 14336), (8, 4096, 14336), (9, 96, 14336)]:
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
        want = ref.linear(x, w, torch.zeros(M, N, dtype=torch.float64))
        mag = (x.double().abs() @ w.double().abs().T).max().item()
        got = ops.linear(x.to(DEV), w.to(DEV), torch.empty(M, N, dtype=torch.float32, device=DEV))
        close(got, want, 1e-6, 4e-7 * mag + 1e-6, f"sliced M{M} N{N} K{K}")


def test_linear_bf16_strided_input(ops, ref):
    """x as a column slice of a wider matrix (row stride larger than K)."""
    g = gen(6)
    wide = torch.randn(9, 512, generator=g).to(torch.bfloat16)
    w = (torch.randn(96, 256, generator=g) / 16).to(torch.bfloat16)
    want = ref.linear(wide[:, 128:384], w, torch.empty(9, 96, dtype=torch.float64))
    got = ops.linear(wide.to(DEV)[:, 128:384], w.to(DEV), torch.empty(9, 96, dtype=torch.float32, device=DEV))
    close(got, want, 1e-5, 1e-5, "strided")


# ---- fused forms of decode steps ----------------------------------------------------------------
FUSED_SHAPES = [(1, 4096, 4096), (1, 64, 136), (8, 6144, 4096), (5, 100, 72), (16, 520, 264), (13, 128, 128), (2, 1000, 4096),
                (16, 4096, 4096), (9, 96, 14336), (3, 256, 20000), (16, 48, 40000),
                # 17 to 64 rows: the slab kernel with the norm folded in
                (17, 128, 128), (64, 6144, 4096), (33, 1000, 4096), (40, 100, 264), (64, 4096, 14336), (24, 96, 1000), (64, 520, 8192)]


def _fused_inputs(M, K, seed):
    g = gen(seed)
    x = torch.randn(M, K, generator=g) * torch.rand(M, 1, generator=g) * 8      # rows of different scale
    nw = 1 + 0.1 * torch.randn(K, generator=g)
    return g, x, nw


@pytest.mark.parametrize("M,N,K", FUSED_SHAPES)
@pytest.mark.parametrize("bias", [False, True])
def test_norm_linear(ops, ref, M, N, K, bias):
    g, x, nw = _fused_inputs(M, K, 30)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g) if bias else None
    want = ref.norm_linear(x, nw, 1e-5, w, torch.empty(M, N, dtype=torch.float64), bias=b)
    got = ops.norm_linear(x.to(DEV), nw.to(DEV), 1e-5, w.to(DEV), torch.empty(M, N, dtype=torch.bfloat16, device=DEV),
                          bias=None if b is None else b.to(DEV))
    # the normed operand is rounded to bfloat16 before the product: sqrt(K) * 2^-9 relative to the row's scale
    close(got, want, 2 * BF16_EPS, 3e-2, f"norm_linear M{M} N{N} K{K}")


@pytest.mark.parametrize("M,inter,K", [(1, 14336, 4096), (1, 176, 64), (8, 432, 160), (13, 1000, 4096), (16, 200, 96), (4, 512, 36000),
                                       (17, 14336, 4096), (64, 176, 64), (40, 432, 160), (33, 1000, 4096), (64, 100, 8192), (64, 14336, 4096)])
def test_norm_gate_up_swiglu(ops, ref, M, inter, K):
    g, x, nw = _fused_inputs(M, K, 31)
    w = (torch.randn(2 * inter, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(2 * inter, generator=g) * 0.1
    want = ref.norm_gate_up_swiglu(x, nw, 1e-6, w, torch.empty(M, inter, dtype=torch.float64), bias=b)
    got = ops.norm_gate_up_swiglu(x.to(DEV), nw.to(DEV), 1e-6, w.to(DEV), torch.empty(M, inter, dtype=torch.bfloat16, device=DEV),
                                  bias=b.to(DEV))
    close(got, want, 2 * BF16_EPS, 4e-2, f"norm_gate_up_swiglu M{M} I{inter} K{K}")


@pytest.mark.parametrize("M,inter,K", [(17, 14336, 4096), (64, 176, 64), (40, 432, 160), (33, 1000, 4096), (24, 200, 96), (64, 36, 8192),
                                       (8, 432, 160), (1, 176, 64)])
def test_gate_up_swiglu(ops, ref, M, inter, K):
    g = gen(46)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(2 * inter, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(2 * inter, generator=g) * 0.1
    want = ref.gate_up_swiglu(x, w, torch.empty(M, inter, dtype=torch.float64), bias=b)
    outs = [ops.gate_up_swiglu(x.to(DEV), w.to(DEV), torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), bias=b.to(DEV))
            for _ in range(3)]
    close(outs[0], want, 2 * BF16_EPS, 2e-2, f"gate_up_swiglu M{M} I{inter} K{K}")
    assert torch.equal(outs[1], outs[0]) and torch.equal(outs[2], outs[0])


@pytest.mark.parametrize("heads,kv_heads,head_dim,rope_dims,page_size,K", [(4, 2, 16, 16, 16, 64), (5, 1, 32, 32, 8, 160),
                                                                           (6, 3, 48, 24, 16, 96), (32, 8, 128, 128, 16, 4096),
                                                                           (2, 2, 16, 0, 16, 64)])
@pytest.mark.parametrize("segs", [[(0, 1)], [(14, 1), (15, 1), (16, 1), (100, 1), (7, 1)], [(5, 3), (40, 2), (127, 1)],
                                  [(3, 17)], [(0, 40), (100, 20)], [(i, 1) for i in range(60, 124)]])
def test_norm_qkv_rope_store(ops, ref, heads, kv_heads, head_dim, rope_dims, page_size, K, segs):
    g, _, _ = _fused_inputs(1, 8, 32)
    rows = sum(n for _, n in segs)
    _, x, nw = _fused_inputs(rows, K, 33)
    positions = 128
    pages_each = positions // page_size
    num_pages = len(segs) * pages_each + 3
    tables = scattered_tables(g, len(segs), pages_each, num_pages)
    row_pos = torch.tensor([p + i for p, n in segs for i in range(n)], dtype=torch.int32)
    row_seg = torch.tensor([s for s, (_, n) in enumerate(segs) for _ in range(n)], dtype=torch.int32)
    row_seg[-1] = -1 if rows > 3 else row_seg[-1]             # a padding row stores nothing
    angle = torch.rand(positions, rope_dims // 2, generator=g, dtype=torch.float64) * 6.28
    cos, sin = torch.cos(angle).float(), torch.sin(angle).float()
    N = (heads + 2 * kv_heads) * head_dim
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g) * 0.1
    k0, v0 = make_pages(g, num_pages, kv_heads, page_size, head_dim, torch.bfloat16)
    k_ref, v_ref = k0.clone(), v0.clone()
    q_ref = ref.norm_qkv_rope_store(x, nw, 1e-5, w, torch.zeros(rows, heads * head_dim, dtype=torch.float64), row_pos, row_seg,
                                    tables, cos, sin, k_ref, v_ref, heads, kv_heads, head_dim, rope_dims, page_size, bias=b)
    k_gpu, v_gpu = k0.to(DEV), v0.to(DEV)
    q_gpu = ops.norm_qkv_rope_store(x.to(DEV), nw.to(DEV), 1e-5, w.to(DEV), torch.zeros(rows, heads * head_dim, dtype=torch.bfloat16, device=DEV),
                                    row_pos.to(DEV), row_seg.to(DEV), tables.to(DEV), cos.to(DEV), sin.to(DEV), k_gpu, v_gpu,
                                    heads, kv_heads, head_dim, rope_dims, page_size, bias=b.to(DEV))
    live = (row_seg >= 0)
    close(q_gpu[live.to(DEV)], q_ref[live], 2 * BF16_EPS, 4e-2, "fused q")
    close(k_gpu, k_ref, 2 * BF16_EPS, 4e-2, "fused k pages")
    close(v_gpu, v_ref, 2 * BF16_EPS, 4e-2, "fused v pages")
    # slots of other tokens keep their bits
    untouched = torch.ones(num_pages, page_size, dtype=torch.bool)
    for r in range(rows):
        if row_seg[r] >= 0:
            untouched[int(tables[int(row_seg[r]), int(row_pos[r]) // page_size]), int(row_pos[r]) % page_size] = False
    assert torch.equal(k_gpu.cpu().permute(0, 3, 1, 2, 4)[untouched], k0.permute(0, 3, 1, 2, 4)[untouched])
    assert torch.equal(v_gpu.cpu().permute(0, 3, 1, 2)[untouched], v0.permute(0, 3, 1, 2)[untouched])
    # reading another entry's cache: queries only
    k2, v2 = k0.to(DEV), v0.to(DEV)
    q2 = ops.norm_qkv_rope_store(x.to(DEV), nw.to(DEV), 1e-5, w.to(DEV), torch.zeros(rows, heads * head_dim, dtype=torch.bfloat16, device=DEV),
                                 row_pos.to(DEV), row_seg.to(DEV), tables.to(DEV), cos.to(DEV), sin.to(DEV), None, None,
                                 heads, kv_heads, head_dim, rope_dims, page_size, bias=b.to(DEV))
    assert torch.equal(q2[live.to(DEV)], q_gpu[live.to(DEV)])


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 4096, 14336), (8, 4096, 4096), (16, 2048, 8192), (5, 160, 432), (13, 64, 176),
                                   (3, 8192, 28672), (8, 320, 40000), (2, 48, 96)])
def test_a_product_prepares_the_norm_that_reads_its_sums(ops, ref, M, N, K):
    """`linear_add_prepare` adds to the residual stream exactly as `linear` does and leaves, for the norm that comes
    next, the rows times the norm's weight in bfloat16 (bit for bit what the norm forms compute themselves) and the rows'
    sums of squares in parts; the gate/up and q/k/v forms fed with that pair give what they give from the float32 rows,
    up to the order in which the squares are added.  Rows of different scale, a width per tile size, K beyond what
    LDS holds (K slices over workgroups), several calls in a row."""
    g = gen(70 + M)
    x = (torch.randn(M, K, generator=g) * 0.5).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g) * 0.1
    resid = torch.randn(M, N, generator=g) * torch.rand(M, 1, generator=g) * 6
    nw = 1 + 0.1 * torch.randn(N, generator=g)
    plain = ops.linear(x.to(DEV), w.to(DEV), resid.clone().to(DEV), bias=b.to(DEV), accumulate=True)
    for _ in range(2):
        summed = resid.clone().to(DEV)
        prepared = ops.linear_add_prepare(x.to(DEV), w.to(DEV), summed, nw.to(DEV), bias=b.to(DEV))
        assert torch.equal(summed, plain)
        assert torch.equal(prepared.x, (summed * nw.to(DEV)).to(torch.bfloat16))
        assert prepared.parts in (N // 16, N // 8)
        squares = prepared.ssq[:M * prepared.parts].view(M, prepared.parts).double().sum(1)
        want = summed.double().pow(2).sum(1)
        assert float(((squares - want).abs() / want).max()) < 1e-6
    # the products behind that norm
    inter = 3 * N // 2 + 8
    wgu = (torch.randn(2 * inter, N, generator=g) / math.sqrt(N)).to(torch.bfloat16).to(DEV)
    bgu = (torch.randn(2 * inter, generator=g) * 0.1).to(DEV)
    own = ops.norm_gate_up_swiglu(summed, nw.to(DEV), 1e-5, wgu, torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), bias=bgu)
    fed = ops.norm_gate_up_swiglu(None, None, 1e-5, wgu, torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), bias=bgu, prepared=prepared)
    want = ref.norm_gate_up_swiglu(summed.cpu(), nw, 1e-5, wgu.cpu(), torch.empty(M, inter, dtype=torch.float64), bias=bgu.cpu())
    close(fed, want, 2 * BF16_EPS, 4e-2, f"gate/up behind a prepared norm M{M} N{N}")
    assert float((fed.float() - own.float()).abs().max()) <= 2 * BF16_EPS * float(own.float().abs().max())
    if N % 64 == 0:
        heads, kv_heads, head_dim, page_size = N // 64, 1, 16, 16
        qkv_rows = (heads + 2) * head_dim
        wq = (torch.randn(qkv_rows, N, generator=g) / math.sqrt(N)).to(torch.bfloat16).to(DEV)
        tables = scattered_tables(g, M, 8, M * 8 + 2).to(DEV)
        row_pos = torch.tensor([(7 * r + 3) % 128 for r in range(M)], dtype=torch.int32, device=DEV)
        row_seg = torch.arange(M, dtype=torch.int32, device=DEV)
        angle = torch.rand(128, head_dim // 2, generator=g, dtype=torch.float64) * 6.28
        cos, sin = torch.cos(angle).float().to(DEV), torch.sin(angle).float().to(DEV)
        k0, v0 = make_pages(g, M * 8 + 2, kv_heads, page_size, head_dim, torch.bfloat16)
        results = []
        for kwargs in ({}, {"prepared": prepared}):
            kp, vp = k0.to(DEV), v0.to(DEV)
            q = ops.norm_qkv_rope_store(summed, nw.to(DEV), 1e-5, wq, torch.zeros(M, heads * head_dim, dtype=torch.bfloat16, device=DEV),
                                        row_pos, row_seg, tables, cos, sin, kp, vp, heads, kv_heads, head_dim, head_dim, page_size, **kwargs)
            results.append((q, kp, vp))
        for got, base in zip(results[1], results[0]):
            assert float((got.float() - base.float()).abs().max()) <= 2 * BF16_EPS * float(base.float().abs().max())
    with pytest.raises(Exception, match="1..128 rows"):
        ops.linear_add_prepare(torch.zeros(129, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV),
                               torch.zeros(129, 32, device=DEV), torch.ones(32, device=DEV))
    with pytest.raises(Exception, match="tile-major copy"):      # beyond 64 rows only from the copy
        ops.linear_add_prepare(torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV),
                               torch.zeros(65, 32, device=DEV), torch.ones(32, device=DEV))
    with pytest.raises(Exception, match="steps of 16"):
        ops.linear_add_prepare(torch.zeros(2, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(24, 64, dtype=torch.bfloat16, device=DEV),
                               torch.zeros(2, 24, device=DEV), torch.ones(24, device=DEV))


@pytest.mark.parametrize("M,heads,kv_heads,head_dim,K,bias", [(1, 32, 8, 128, 4096, False), (8, 32, 8, 128, 4096, True), (16, 32, 8, 128, 4096, False),
                                                              (5, 6, 2, 80, 2048, True), (11, 3, 1, 16, 1024, True), (9, 8, 4, 64, 3072, False)])
def test_qkv_of_up_to_16_rows_streams_the_tile_major_copy(ops, ref, M, heads, kv_heads, head_dim, K, bias):
    """Up to 16 rows the q/k/v product behind a prepared norm reads whole 16-row tiles from the tile-major copy where
    there is one and the launch fits it; without the copy (or with the switch off) it reads the matrix, in 8-row tiles
    where those fill the device better.  All of them against the form that norms the float32 rows itself."""
    g = gen(300 + M + heads)
    page_size = 16
    rows = (torch.randn(M, K, generator=g) * torch.rand(M, 1, generator=g) * 4).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
    n = (heads + 2 * kv_heads) * head_dim
    wq = (torch.randn(n, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    bq = (torch.randn(n, generator=g) * 0.1).to(DEV) if bias else None
    prepared = ops.prepare_norm(rows, nw)
    tables = scattered_tables(g, M, 8, M * 8 + 2).to(DEV)
    row_pos = torch.tensor([(7 * r + 3) % 128 for r in range(M)], dtype=torch.int32, device=DEV)
    row_seg = torch.arange(M, dtype=torch.int32, device=DEV)
    angle = torch.rand(128, head_dim // 2, generator=g, dtype=torch.float64) * 6.28
    cos, sin = torch.cos(angle).float().to(DEV), torch.sin(angle).float().to(DEV)
    k0, v0 = make_pages(g, M * 8 + 2, kv_heads, page_size, head_dim, torch.bfloat16)

    def product(**kwargs):
        kp, vp = k0.to(DEV), v0.to(DEV)
        q = ops.norm_qkv_rope_store(rows, nw, 1e-5, wq, torch.zeros(M, heads * head_dim, dtype=torch.bfloat16, device=DEV), row_pos, row_seg,
                                    tables, cos, sin, kp, vp, heads, kv_heads, head_dim, head_dim, page_size, bias=bq, **kwargs)
        return q, kp, vp

    base = product()
    without = product(prepared=prepared)
    assert ops.tile_for_decode(wq) == (K % 1024 == 0)
    with_copy = product(prepared=prepared)
    ops.set_option("linear.resident_tiles", 0)
    try:
        switched_off = product(prepared=prepared)
    finally:
        ops.set_option("linear.resident_tiles", 1)
    for a, b in zip(switched_off, without):
        assert torch.equal(a, b)
    for other in (without, with_copy):
        for got, want in zip(other, base):
            assert float((got.float() - want.float()).abs().max()) <= 2 * BF16_EPS * float(want.float().abs().max())


@pytest.mark.parametrize("M,N,K", [(17, 4096, 4096), (64, 4096, 14336), (33, 1024, 2048), (48, 2048, 1024), (64, 2048, 8192)])
def test_prepared_norms_of_17_to_64_rows(ops, ref, M, N, K):
    """Steps of 17 to 64 rows run the same five kernels a layer as smaller ones, on the kernels that pass the
    activations through LDS in chunks and read the tile-major copies: the sum into the residual stream prepares the
    next norm, the gate/up and q/k/v products take the prepared rows and scale their sums by the row's norm.  Against
    the float64 results, against the same forms fed with the float32 rows (another kernel), and with the preparation
    made by `prepare_norm` (a model's first layer)."""
    g = gen(170 + M)
    x = (torch.randn(M, K, generator=g) * 0.5).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    resid = (torch.randn(M, N, generator=g) * torch.rand(M, 1, generator=g) * 6).to(DEV)
    nw = (1 + 0.1 * torch.randn(N, generator=g)).to(DEV)
    few = min(M, ops.CHUNK_ROWS)                             # the kernels take up to 64 rows, steps use them up to CHUNK_ROWS
    assert ops.tile_for_decode(w) and ops.fused_form(few, K, w) == "chunks" and ops.prepares_norm(few, N, w)
    assert ops.fused_form(few, K, w.clone()) is None         # no copy: the library's products and the separate kernels serve
    assert ops.fused_form(ops.CHUNK_ROWS + 1, K, w) is None
    summed = resid.clone()
    prepared = ops.linear_add_prepare(x, w, summed, nw)
    want = ref.linear(x.cpu(), w.cpu(), resid.double().cpu(), accumulate=True)
    mag = (x.double().abs() @ w.double().abs().T).max().item()
    close(summed, want, 1e-6, 4e-7 * mag + 1e-6, f"sum M{M} N{N} K{K}")
    assert torch.equal(summed, ops.linear(x, w, resid.clone(), accumulate=True))
    assert torch.equal(prepared.x, (summed * nw).to(torch.bfloat16)) and prepared.parts == N // 16
    squares = prepared.ssq[:M * prepared.parts].view(M, prepared.parts).double().sum(1)
    assert float(((squares - summed.double().pow(2).sum(1)).abs() / summed.double().pow(2).sum(1)).max()) < 1e-6
    first = ops.prepare_norm(summed, nw)
    assert torch.equal(first.x, prepared.x) and first.parts == 1
    assert float(((first.ssq.double() - squares).abs() / squares).max()) < 1e-6
    # the products behind that norm
    inter = 3 * N // 2 + 8
    wgu = (torch.randn(2 * inter, N, generator=g) / math.sqrt(N)).to(torch.bfloat16).to(DEV)
    bgu = (torch.randn(2 * inter, generator=g) * 0.1).to(DEV)
    assert ops.tile_for_decode(wgu, gate_up=True) and ops.fused_form(few, N, wgu, gate_up=True) == "chunks"
    want = ref.norm_gate_up_swiglu(summed.cpu(), nw.cpu(), 1e-5, wgu.cpu(), torch.empty(M, inter, dtype=torch.float64), bias=bgu.cpu())
    own = ops.norm_gate_up_swiglu(summed, nw, 1e-5, wgu, torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), bias=bgu)
    for pair in (prepared, first):
        fed = ops.norm_gate_up_swiglu(None, None, 1e-5, wgu, torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), bias=bgu, prepared=pair)
        close(fed, want, 2 * BF16_EPS, 4e-2, f"gate/up behind a prepared norm M{M} N{N}")
        assert float((fed.float() - own.float()).abs().max()) <= 2 * BF16_EPS * float(own.float().abs().max())
    heads, kv_heads, head_dim, page_size = N // 64, 2, 16, 16
    qkv_rows = (heads + 2 * kv_heads) * head_dim
    wq = (torch.randn(qkv_rows, N, generator=g) / math.sqrt(N)).to(torch.bfloat16).to(DEV)
    assert ops.tile_for_decode(wq)
    tables = scattered_tables(g, M, 8, M * 8 + 2).to(DEV)
    row_pos = torch.tensor([(7 * r + 3) % 128 for r in range(M)], dtype=torch.int32, device=DEV)
    row_seg = torch.arange(M, dtype=torch.int32, device=DEV)
    row_seg[M // 2] = -1                                   # a padding row stores nothing
    angle = torch.rand(128, head_dim // 2, generator=g, dtype=torch.float64) * 6.28
    cos, sin = torch.cos(angle).float().to(DEV), torch.sin(angle).float().to(DEV)
    k0, v0 = make_pages(g, M * 8 + 2, kv_heads, page_size, head_dim, torch.bfloat16)
    results = []
    for kwargs in ({}, {"prepared": prepared}, {"prepared": first}):
        kp, vp = k0.to(DEV), v0.to(DEV)
        q = ops.norm_qkv_rope_store(summed, nw, 1e-5, wq, torch.zeros(M, heads * head_dim, dtype=torch.bfloat16, device=DEV),
                                    row_pos, row_seg, tables, cos, sin, kp, vp, heads, kv_heads, head_dim, head_dim, page_size, **kwargs)
        results.append((q, kp, vp))
    live = row_seg >= 0
    for other in results[1:]:
        for got, base in zip(other, results[0]):
            got, base = (got[live], base[live]) if got.shape[0] == M else (got, base)
            assert float((got.float() - base.float()).abs().max()) <= 2 * BF16_EPS * float(base.float().abs().max())
    assert torch.equal(results[1][0][~live], torch.zeros_like(results[1][0][~live]))
    with pytest.raises(Exception, match="tile-major copy"):
        ops.norm_gate_up_swiglu(None, None, 1e-5, wgu.clone(), torch.empty(M, inter, dtype=torch.bfloat16, device=DEV), prepared=prepared)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,inter", [(1, 176), (13, 432), (3, 14336)])
def test_swiglu(ops, ref, dtype, rows, inter):
    g = gen(7)
    gu = (torch.randn(rows, 2 * inter, generator=g) * 3).to(dtype)
    gu[0, 0] = 0.0
    gu[0, 1] = 30.0
    want = ref.swiglu(gu, torch.empty(rows, inter, dtype=torch.float64))
    got = ops.swiglu(gu.to(DEV), torch.empty(rows, inter, dtype=dtype, device=DEV))
    tol = 2e-6 if dtype == torch.float32 else BF16_EPS
    close(got, want, tol, 1e-7, "swiglu")


# ---------------------------------------------------------------------------------------------
def make_pages(g, num_pages, kv_heads, page_size, head_dim, dtype):
    """Pages as the kernels lay them out: keys chunk by chunk [page][kv_head][head_dim / 8][token][8], values
    [page][kv_head][head_dim][token]."""
    k = torch.randn(num_pages, kv_heads, head_dim // 8, page_size, 8, generator=g).to(dtype)
    v = torch.randn(num_pages, kv_heads, head_dim, page_size, generator=g).to(dtype)
    return k, v


def scattered_tables(g, segments, pages_each, num_pages):
    perm = torch.randperm(num_pages, generator=g)[: segments * pages_each].to(torch.int32)
    return perm.view(segments, pages_each).contiguous()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,head_dim,rope_dims,pairing,page_size",
                         [(4, 2, 16, 16, 0, 16), (5, 1, 32, 32, 0, 8), (6, 3, 48, 24, 0, 16), (8, 2, 64, 64, 1, 16),
                          (32, 8, 128, 128, 0, 16), (2, 2, 16, 0, 0, 4)])
def test_rope_kv_store(ops, ref, dtype, heads, kv_heads, head_dim, rope_dims, pairing, page_size):
    _rope_case(ops, ref, dtype, heads, kv_heads, head_dim, rope_dims, pairing, page_size,
               [(0, 5), (37, 1), (page_size - 1, 3), (100, 17)], 128)


@pytest.mark.parametrize("heads,kv_heads,head_dim,rope_dims,page_size", [(8, 2, 64, 64, 16), (32, 8, 128, 128, 16), (4, 2, 16, 8, 8),
                                                                         (6, 3, 48, 24, 32)])
def test_rope_kv_store_prompt_portions(ops, ref, heads, kv_heads, head_dim, rope_dims, page_size):
    """Hundreds of rows: runs of 8 tokens that start at a multiple of 8 store their values 16 bytes at a time; runs
    that start elsewhere, single rows and the ends of portions take the other way."""
    _rope_case(ops, ref, torch.bfloat16, heads, kv_heads, head_dim, rope_dims, 1, page_size,
               [(0, 300), (37, 1), (13, 40), (8, 64), (509, 3)], 512)


def _rope_case(ops, ref, dtype, heads, kv_heads, head_dim, rope_dims, pairing, page_size, segs, positions):
    g = gen(8)
    rows = sum(n for _, n in segs)             # segs: (first position, rows)
    pages_each = positions // page_size
    num_pages = len(segs) * pages_each + 3
    tables = scattered_tables(g, len(segs), pages_each, num_pages)
    row_pos = torch.tensor([p + i for p, n in segs for i in range(n)], dtype=torch.int32)
    row_seg = torch.tensor([s for s, (_, n) in enumerate(segs) for _ in range(n)], dtype=torch.int32)
    half = rope_dims // 2
    angle = torch.rand(positions, half, generator=g, dtype=torch.float64) * 6.28
    cos, sin = torch.cos(angle).float(), torch.sin(angle).float()
    qkv = torch.randn(rows, (heads + 2 * kv_heads) * head_dim, generator=g).to(dtype)
    k0, v0 = make_pages(g, num_pages, kv_heads, page_size, head_dim, dtype)
    q_ref, k_ref, v_ref = qkv.clone(), k0.clone(), v0.clone()
    ref.rope_kv_store(q_ref, row_pos, row_seg, tables, cos, sin, k_ref, v_ref, heads, kv_heads, head_dim, rope_dims,
                      pairing, page_size)
    q_gpu, k_gpu, v_gpu = qkv.to(DEV), k0.to(DEV), v0.to(DEV)
    ops.rope_kv_store(q_gpu, row_pos.to(DEV), row_seg.to(DEV), tables.to(DEV), cos.to(DEV), sin.to(DEV), k_gpu, v_gpu,
                      heads, kv_heads, head_dim, rope_dims, pairing, page_size)
    tol = 1e-6 if dtype == torch.float32 else BF16_EPS
    width = heads * head_dim
    close(q_gpu[:, :width], q_ref[:, :width], tol, tol, "rotated q")
    close(k_gpu, k_ref, tol, tol, "k pages")
    assert torch.equal(v_gpu.cpu(), v_ref), "v pages"
    # a layer that reads another layer's cache rotates q and leaves the pages alone
    q2, k2, v2 = qkv.to(DEV), k0.to(DEV), v0.to(DEV)
    ops.rope_kv_store(q2, row_pos.to(DEV), row_seg.to(DEV), tables.to(DEV), cos.to(DEV), sin.to(DEV), None, None,
                      heads, kv_heads, head_dim, rope_dims, pairing, page_size)
    assert torch.equal(q2[:, :width], q_gpu[:, :width]) and torch.equal(k2.cpu(), k0) and torch.equal(v2.cpu(), v0)


# ---------------------------------------------------------------------------------------------
def attention_case(ops, ref, dtype, heads, kv_heads, head_dim, page_size, segs, window, seed, fast=True, spike=False,
                   bound=None, calls=1, mark_single_rows=True, slopes=None):
    """segs: (first position, rows) per segment.  bound: the context bound handed to the kernel (a decode graph's
    is larger than any context of the step); calls: launches in a row, which must give the same bits."""
    g = gen(seed)
    rows = sum(n for _, n in segs)
    max_context = max(p + n for p, n in segs)
    pages_each = -(-max_context // page_size)
    num_pages = len(segs) * pages_each + 2
    tables = scattered_tables(g, len(segs), pages_each, num_pages)
    row_pos = torch.tensor([p + i for p, n in segs for i in range(n)], dtype=torch.int32)
    row_seg = torch.tensor([s for s, (_, n) in enumerate(segs) for _ in range(n)], dtype=torch.int32)
    seg_start = torch.tensor(np.cumsum([0] + [n for _, n in segs]), dtype=torch.int32)
    k, v = make_pages(g, num_pages, kv_heads, page_size, head_dim, dtype)
    stride = (heads + 2 * kv_heads) * head_dim
    qkv = torch.randn(rows, stride, generator=g).to(dtype)
    if spike:
        # one far key stands out for the last row of every segment: a wrong page, a wrong slot or a
        # key that a split loses changes the output completely
        r = 0
        for s, (p, n) in enumerate(segs):
            r += n
            pos = p + n - 1
            lo = max(0, pos + 1 - window) if window else 0
            far = lo + (pos - lo) // 7
            page, off = int(tables[s, far // page_size]), far % page_size
            for h in range(heads):
                q = qkv[r - 1, h * head_dim:(h + 1) * head_dim].float()
                k[page, h // (heads // kv_heads), :, off, :] = (q * (12.0 / q.norm() ** 2 * math.sqrt(head_dim))).to(dtype).view(-1, 8)
    q = qkv[:, : heads * head_dim]
    scale = head_dim ** -0.5
    want = ref.attention(q, k, v, tables, row_pos, row_seg, seg_start, torch.empty(rows, heads * head_dim, dtype=torch.float64),
                         heads, kv_heads, head_dim, page_size, scale, window, max_context, head_slopes=slopes)
    if window:
        # pages that lie wholly before the window of a segment's first row have been given back: their table entries
        # are -1, and a kernel that looked at them would read outside the pages
        tables = tables.clone()
        for s, (p, n) in enumerate(segs):
            tables[s, : max(0, p + 1 - window) // page_size] = -1
    uniform = int(all(n == 1 for _, n in segs))
    single_from = len(segs)
    while single_from > 0 and segs[single_from - 1][1] == 1:
        single_from -= 1
    if not mark_single_rows:
        single_from = 0 if uniform else len(segs)
    ops.set_fast_kernels(fast)
    try:
        bound = max_context if bound is None else bound
        nbytes = max(ops.attention_workspace_bytes(n, heads, kv_heads, head_dim, bound) for n in {rows, len(segs) - single_from} if n > 0)
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=DEV)
        args = (qkv.to(DEV)[:, : heads * head_dim], k.to(DEV), v.to(DEV), tables.to(DEV), row_pos.to(DEV), row_seg.to(DEV),
                seg_start.to(DEV))
        got = None
        for _ in range(calls):
            out = ops.attention(*args, torch.empty(rows, heads * head_dim, dtype=dtype, device=DEV),
                                heads, kv_heads, head_dim, page_size, scale, window, bound, single_from=single_from, workspace=ws,
                                head_slopes=None if slopes is None else slopes.to(DEV))
            assert got is None or torch.equal(out, got), "two launches of the same attention differ"
            got = out
    finally:
        ops.set_fast_kernels(True)
    if dtype == torch.float32:
        close(got, want, 1e-5, 1e-5, "attention f32")
    else:
        close(got, want, 2 * BF16_EPS, 1.5e-2, "attention bf16")    # probabilities are rounded to bfloat16 before PV
    return got


SHAPES = [(4, 2, 16, 16), (5, 1, 32, 8), (6, 3, 48, 16), (8, 2, 64, 16), (32, 8, 128, 16), (8, 8, 64, 32), (16, 1, 128, 16)]
DECODE_SEGS = [[(0, 1)], [(14, 1), (15, 1), (16, 1), (17, 1)], [(126, 1), (127, 1), (128, 1), (1, 1), (63, 1)],
               [(999, 1), (5, 1), (640, 1)]]
CHUNK_SEGS = [[(0, 5)], [(0, 64)], [(0, 70)], [(100, 17), (37, 1), (0, 33)], [(3, 70), (200, 2), (15, 2), (16, 1)],
              [(0, 300)], [(250, 50), (0, 1)], [(100, 120), (0, 40), (37, 1)], [(0, 2048)]]


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", SHAPES)
@pytest.mark.parametrize("segs", DECODE_SEGS + CHUNK_SEGS)
def test_attention_f32(ops, ref, heads, kv_heads, head_dim, page_size, segs):
    attention_case(ops, ref, torch.float32, heads, kv_heads, head_dim, page_size, segs, None, 9)


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", SHAPES)
@pytest.mark.parametrize("segs", DECODE_SEGS + CHUNK_SEGS)
def test_attention_bf16(ops, ref, heads, kv_heads, head_dim, page_size, segs):
    attention_case(ops, ref, torch.bfloat16, heads, kv_heads, head_dim, page_size, segs, None, 10)


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(4, 2, 16, 16), (8, 2, 64, 16), (32, 8, 128, 16)])
@pytest.mark.parametrize("segs", [DECODE_SEGS[2], DECODE_SEGS[3], CHUNK_SEGS[3], CHUNK_SEGS[4]])
def test_attention_bf16_plain_kernel(ops, ref, heads, kv_heads, head_dim, page_size, segs):
    attention_case(ops, ref, torch.bfloat16, heads, kv_heads, head_dim, page_size, segs, None, 11, fast=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(6, 3, 48, 16), (8, 2, 64, 16), (32, 8, 128, 16), (5, 1, 32, 8)])
@pytest.mark.parametrize("window", [1, 24, 100])
@pytest.mark.parametrize("segs", [DECODE_SEGS[1], DECODE_SEGS[3], CHUNK_SEGS[3], CHUNK_SEGS[4], CHUNK_SEGS[5], CHUNK_SEGS[6],
                                  CHUNK_SEGS[7]])
def test_attention_window(ops, ref, dtype, heads, kv_heads, head_dim, page_size, window, segs):
    attention_case(ops, ref, dtype, heads, kv_heads, head_dim, page_size, segs, window, 12)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("segs,window", [([(900, 1), (333, 1)], None), ([(700, 90), (0, 200)], None), ([(900, 1)], 500),
                                          ([(640, 64)], 300)])
def test_attention_far_key_stands_out(ops, ref, dtype, segs, window):
    attention_case(ops, ref, dtype, 8, 2, 64, 16, segs, window, 13, spike=True)
    attention_case(ops, ref, dtype, 32, 8, 128, 16, segs, window, 14, spike=True)


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(8, 2, 64, 16), (32, 8, 128, 16), (8, 8, 64, 32), (16, 1, 128, 16)])
@pytest.mark.parametrize("segs,window", [(CHUNK_SEGS[3], None), (CHUNK_SEGS[4], None), (CHUNK_SEGS[5], None), (CHUNK_SEGS[7], 100),
                                          ([(640, 64)], 300)])
def test_attention_bf16_tile_kernel_of_64_rows(ops, ref, heads, kv_heads, head_dim, page_size, segs, window):
    """Heads of 64 and 128 go to the 128-row kernel by default; the 64-row kernel serves them when that is switched off."""
    ops.set_option("attention.tile32", 0)
    try:
        attention_case(ops, ref, torch.bfloat16, heads, kv_heads, head_dim, page_size, segs, window, 17, spike=True)
    finally:
        ops.set_option("attention.tile32", 1)


@pytest.mark.parametrize("rows", [128, 256])
@pytest.mark.parametrize("prefill_parts", [1, 0])
@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(8, 2, 64, 16), (32, 8, 128, 16), (8, 8, 64, 32), (16, 1, 128, 16), (6, 3, 64, 8)])
@pytest.mark.parametrize("segs,window", [(CHUNK_SEGS[3], None), (CHUNK_SEGS[4], None), (CHUNK_SEGS[5], None), (CHUNK_SEGS[7], 100),
                                          ([(640, 64)], 300), ([(0, 700), (1500, 40), (3, 300)], None), ([(0, 1100)], None)])
def test_attention_bf16_row_tiles_of_128_and_256(ops, ref, rows, prefill_parts, heads, kv_heads, head_dim, page_size, segs, window):
    """The prompt kernel takes 128 rows a workgroup or 256 (one workgroup a compute unit: a key fetched from L2 serves
    twice the rows); a launch picks by how many row tiles it has, `attention.tile32_rows` by hand.  Both against the plain
    reference, with and without row tiles shared between workgroups, with a far key that stands out."""
    ops.set_option("attention.tile32_rows", rows)
    ops.set_option("attention.prefill_parts", prefill_parts)
    try:
        attention_case(ops, ref, torch.bfloat16, heads, kv_heads, head_dim, page_size, segs, window, 23, spike=True, calls=2)
    finally:
        ops.set_option("attention.tile32_rows", 0)
        ops.set_option("attention.prefill_parts", 1)
    torch.cuda.synchronize()
    from fllm_amd.kernels import Ops
    counters = Ops._workspaces[torch.cuda.current_device()][: 64 * 1024]
    assert int(counters.to(torch.int64).sum()) == 0


@pytest.mark.parametrize("fused_merge", [1, 0])
@pytest.mark.parametrize("heads,kv_heads,head_dim,page_size", [(8, 2, 64, 16), (32, 8, 128, 16), (5, 1, 32, 8)])
@pytest.mark.parametrize("segs,bound,window", [([(999, 1), (5, 1), (640, 1)], 2048, None), ([(1100, 1)], 4096, None),
                                                ([(300, 1), (2500, 1)], 8192, 700), ([(0, 1)], 1024, None)])
def test_attention_decode_split_contexts(ops, ref, fused_merge, heads, kv_heads, head_dim, page_size, segs, bound, window):
    """A decode step splits its contexts over workgroups by the bound of the step, not by the contexts themselves:
    splits without keys, one split alone, and the merge by the last split or by a second kernel."""
    ops.set_option("attention.fused_merge", fused_merge)
    try:
        attention_case(ops, ref, torch.bfloat16, heads, kv_heads, head_dim, page_size, segs, window, 16, spike=True,
                       bound=bound, calls=3)
    finally:
        ops.set_option("attention.fused_merge", 1)


@pytest.mark.parametrize("segs,bound,window", [([(20000, 1), (70, 1)], 32768, None), ([(40000, 1)], 65536, None),
                                                ([(16380, 6)], None, None), ([(30000, 3)], None, 4096)])
def test_attention_long_contexts(ops, ref, segs, bound, window):
    """Tens of thousands of keys: many splits of a decode row, many tiles of a prompt portion, page tables of
    thousands of entries; one far key stands out, so a lost split or a wrong page changes the output."""
    attention_case(ops, ref, torch.bfloat16, 32, 8, 128, 16, segs, window, 18, spike=True, bound=bound)
    attention_case(ops, ref, torch.bfloat16, 8, 2, 64, 16, segs, window, 19, spike=True, bound=bound)


@pytest.mark.parametrize("prefill_parts", [1, 0])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [(32, 8, 128), (8, 2, 64), (6, 3, 64), (16, 1, 128)])
@pytest.mark.parametrize("segs,bound", [([(1500, 40), (0, 700), (5000, 3)], None), ([(0, 1100)], None), ([(600, 70), (0, 2)], 8192),
                                        ([(513, 31), (1000, 33)], 1100), ([(0, 2048)], None)])
def test_attention_prompt_portions_share_long_row_tiles(ops, ref, prefill_parts, heads, kv_heads, head_dim, segs, bound):
    """Few rows over long contexts, and whole prompts (row tiles of every length, the long ones shared in halves): the
    keys of a row tile are dealt out to several workgroups, by the bound of the
    step (parts without keys leave at once), and the one that arrives last adds the parts up: the same bits in
    every launch, and the counters they meet at are left at zero."""
    ops.set_option("attention.prefill_parts", prefill_parts)
    try:
        attention_case(ops, ref, torch.bfloat16, heads, kv_heads, head_dim, 16, segs, None, 21, spike=True, bound=bound, calls=3)
    finally:
        ops.set_option("attention.prefill_parts", 1)
    torch.cuda.synchronize()
    from fllm_amd.kernels import Ops
    counters = Ops._workspaces[torch.cuda.current_device()][: 64 * 1024]
    assert int(counters.to(torch.int64).sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [(8, 2, 128), (5, 1, 32), (6, 3, 48)])
@pytest.mark.parametrize("segs,window", [([(0, 70), (300, 1), (37, 1)], None), ([(250, 50), (900, 1)], 100)])
def test_attention_with_scores_biased_by_distance(ops, ref, dtype, heads, kv_heads, head_dim, segs, window):
    """A slope per head times (key position - row position) on every score, as a position encoding that biases
    scores asks for: steep slopes, so that a bias left out, of the wrong sign or of the wrong head changes the
    result (the far key that stands out without the bias no longer does with it)."""
    slopes = torch.tensor([0.05 * (1 + h % 4) for h in range(heads)], dtype=torch.float32)
    biased = attention_case(ops, ref, dtype, heads, kv_heads, head_dim, 16, segs, window, 31, spike=True, calls=2, slopes=slopes)
    plain = attention_case(ops, ref, dtype, heads, kv_heads, head_dim, 16, segs, window, 31, spike=True)
    assert (biased.float() - plain.float()).abs().max() > 0.05
    from fllm_amd.kernels import KernelError
    q = torch.zeros(1, heads * head_dim, dtype=dtype, device=DEV)
    pages = torch.zeros(2, kv_heads, head_dim // 8, 16, 8, dtype=dtype, device=DEV)
    ints = lambda *v: torch.tensor(v, dtype=torch.int32, device=DEV)
    with pytest.raises(KernelError, match="head_slopes"):        # one slope too few
        ops.attention(q, pages, pages.view(2, kv_heads, head_dim, 16), ints(0).view(1, 1), ints(0), ints(0), ints(0, 1),
                      torch.empty_like(q), heads, kv_heads, head_dim, 16, 1.0, None, 1, head_slopes=slopes[:-1].to(DEV))


@pytest.mark.parametrize("mark_single_rows", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [(32, 8, 128), (8, 2, 64), (5, 1, 32), (6, 3, 48)])
@pytest.mark.parametrize("segs,window", [([(0, 300), (5000, 1), (37, 1), (999, 1)], None), ([(100, 17), (0, 33), (640, 1)], None),
                                         ([(3, 70), (700, 2), (2000, 1), (15, 1), (0, 1)], None), ([(250, 50), (900, 1), (30, 1)], 100)])
def test_attention_portions_beside_single_rows(ops, ref, mark_single_rows, dtype, heads, kv_heads, head_dim, segs, window):
    """Portions of prompts with single rows behind them, as a step of the engine lays them out: the single rows go
    to the kernel that splits long contexts when the caller says where they begin, and to the tile kernel with the
    portions when it does not; either way every row is right."""
    attention_case(ops, ref, dtype, heads, kv_heads, head_dim, 16, segs, window, 24, spike=True, calls=2,
                   mark_single_rows=mark_single_rows)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_row_is_the_same_alone_and_in_a_batch(ops, dtype):
    """The bits of a row do not depend on the batch around it: a portion of 17 rows alone and with two other segments
    in the step, on the same pages with the same table."""
    g = gen(15)
    heads, kv_heads, head_dim, page_size = 8, 2, 64, 16
    segs = [(100, 17), (37, 1), (0, 33)]
    pages_each = 8
    num_pages = 3 * pages_each + 2
    tables = scattered_tables(g, 3, pages_each, num_pages)
    k, v = make_pages(g, num_pages, kv_heads, page_size, head_dim, dtype)
    q = torch.randn(51, heads * head_dim, generator=g).to(dtype)
    scale = head_dim ** -0.5

    def run(count):
        these = segs[:count]
        rows = sum(n for _, n in these)
        row_pos = torch.tensor([p + i for p, n in these for i in range(n)], dtype=torch.int32)
        row_seg = torch.tensor([s for s, (_, n) in enumerate(these) for _ in range(n)], dtype=torch.int32)
        seg_start = torch.tensor(np.cumsum([0] + [n for _, n in these]), dtype=torch.int32)
        bound = max(p + n for p, n in these)
        ws = torch.empty(max(1, ops.attention_workspace_bytes(rows, heads, kv_heads, head_dim, bound)), dtype=torch.uint8, device=DEV)
        return ops.attention(q[:rows].to(DEV), k.to(DEV), v.to(DEV), tables[:count].contiguous().to(DEV), row_pos.to(DEV),
                             row_seg.to(DEV), seg_start.to(DEV), torch.empty(rows, heads * head_dim, dtype=dtype, device=DEV),
                             heads, kv_heads, head_dim, page_size, scale, None, bound, single_from=count, workspace=ws)

    together, alone = run(3), run(1)
    assert together.shape[0] == 51 and alone.shape[0] == 17
    assert torch.equal(together[:17], alone), "a row's bits changed with its neighbours"


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("rows,vocab", [(1, 256), (5, 1000), (3, 128256)])
def test_argmax(ops, rows, vocab):
    g = gen(16)
    logits = torch.randn(rows, vocab, generator=g)
    logits[0, 7] = logits[0, vocab - 3] = 50.0          # a tie: the first index wins
    logits[rows - 1, 3] = float("nan")
    logits[rows - 1, 4] = float("inf")
    got = ops.argmax(logits.to(DEV), torch.empty(rows, dtype=torch.int32, device=DEV)).cpu()
    for r in range(rows):
        row = logits[r].numpy()
        want = plain_llama.greedy(np.where(np.isfinite(row), row, -np.inf))
        assert int(got[r]) == want
    assert int(got[0]) == 7


def test_sample_matches_the_plain_sampler(ops):
    from fllm_amd.sampling import SampleRequest, SamplingParams, pack_rows
    g = gen(17)
    vocab = 1000
    cases = [SamplingParams(temperature=0.8), SamplingParams(temperature=1.0, top_k=5),
             SamplingParams(temperature=0.7, top_p=0.9), SamplingParams(temperature=1.3, top_k=50, top_p=0.5),
             SamplingParams(temperature=0.0), SamplingParams(temperature=0.8, top_p=0.01),
             SamplingParams(temperature=1.0, min_p=0.05), SamplingParams(temperature=1.5, top_k=40, min_p=0.2, top_p=0.8),
             SamplingParams(temperature=0.9, min_p=0.3, top_p=0.6), SamplingParams(temperature=0.7, min_p=1.0)]
    logits = torch.randn(len(cases), vocab, generator=g) * 2.0
    for draw in range(6):
        reqs = [SampleRequest(p, seed=1234 + i, draw=draw) for i, p in enumerate(cases)]
        out = torch.empty(len(cases), dtype=torch.int32, device=DEV)
        ops.sample(logits.to(DEV), torch.empty(len(cases), vocab, device=DEV), pack_rows(reqs).to(DEV), out)
        for i, p in enumerate(cases):
            want = plain_llama.device_sample(logits[i].numpy(), p.temperature, p.top_k, p.top_p, 1234 + i, draw, p.min_p)
            assert int(out[i]) == want, (draw, i)


@pytest.mark.parametrize("vocab", [50000, 128256])
def test_sample_thresholds_on_wide_vocabularies(ops, vocab):
    """Thresholds among the few largest logits, thresholds further from the maximum than the sampler's histogram
    reaches, ties at the threshold, flat rows, rows with holes: the token is the plain sampler's in every draw."""
    from fllm_amd.sampling import SampleRequest, SamplingParams, pack_rows
    g = gen(23)
    rows = {
        "normal": torch.randn(vocab, generator=g) * 3.0,
        "wide": torch.randn(vocab, generator=g) * 60.0,                      # thresholds far below the maximum
        "flat": torch.zeros(vocab),                                          # all tied
        "steps": torch.randint(0, 12, (vocab,), generator=g).float() * 0.5,  # many ties at every level
        "holes": torch.randn(vocab, generator=g) * 2.0,
        "peak": torch.randn(vocab, generator=g),
    }
    rows["holes"][::3] = float("-inf")
    rows["holes"][5] = float("nan")
    rows["holes"][11] = float("inf")
    rows["peak"][vocab - 7] = 30.0
    cases = [SamplingParams(temperature=0.8), SamplingParams(temperature=1.0, top_k=1), SamplingParams(temperature=0.6, top_k=5),
             SamplingParams(temperature=1.1, top_k=64), SamplingParams(temperature=1.0, top_k=vocab - 1),
             SamplingParams(temperature=0.7, top_p=0.01), SamplingParams(temperature=1.0, top_p=0.5),
             SamplingParams(temperature=2.5, top_p=0.9), SamplingParams(temperature=4.0, top_p=0.999),
             SamplingParams(temperature=1.3, top_k=50, top_p=0.5), SamplingParams(temperature=0.9, top_k=2000, top_p=0.95),
             SamplingParams(temperature=1.0, min_p=0.1), SamplingParams(temperature=3.0, min_p=0.001),       # a long list
             SamplingParams(temperature=3.0, min_p=0.002, top_p=0.9), SamplingParams(temperature=1.2, top_k=3000, min_p=0.01, top_p=0.9),
             SamplingParams(temperature=40.0, min_p=1e-30)]                                               # further than the histogram reaches
    for name, row in rows.items():
        logits = row.view(1, vocab).expand(len(cases), vocab).contiguous()
        for draw in range(2):
            reqs = [SampleRequest(p, seed=99 + i, draw=draw) for i, p in enumerate(cases)]
            out = torch.empty(len(cases), dtype=torch.int32, device=DEV)
            ops.sample(logits.to(DEV), torch.empty(len(cases), vocab, device=DEV), pack_rows(reqs).to(DEV), out)
            for i, p in enumerate(cases):
                want = plain_llama.device_sample(row.numpy(), p.temperature, p.top_k, p.top_p, 99 + i, draw, p.min_p)
                assert int(out[i]) == want, (name, draw, i)


@pytest.mark.parametrize("vocab", [1000, 128256])
def test_sample_rows_that_draw_from_all_tokens_share_workgroups(ops, vocab):
    """Rows with a temperature and no filter are drawn by several workgroups each (wide vocabularies) in launches of
    their own; what the caller says it knows of the rows (`kinds`) changes no token, rows of both kinds in one call
    are each the plain sampler's, and a row without a finite logit gives token 0."""
    from fllm_amd.sampling import SampleRequest, SamplingParams, pack_rows
    g = gen(29)
    plain = [SamplingParams(temperature=t) for t in (0.3, 1.0, 2.5, 1.0)]
    other = [SamplingParams(temperature=0.9, top_k=7), SamplingParams(temperature=0.0), SamplingParams(temperature=1.2, top_p=0.8)]
    logits = torch.randn(len(plain) + len(other), vocab, generator=g) * 2.5
    logits[3] = float("-inf")
    logits[1, ::5] = float("nan")

    def draw(rows, params, kinds, d):
        reqs = [SampleRequest(p, seed=70 + i, draw=d) for i, p in zip(rows, params)]
        out = torch.full((len(rows),), -1, dtype=torch.int32, device=DEV)
        ops.sample(logits[rows].to(DEV), torch.empty(len(rows), vocab, device=DEV), pack_rows(reqs).to(DEV), out, kinds)
        return out.cpu().tolist()

    for d in range(3):
        want = [plain_llama.device_sample(logits[i].numpy(), p.temperature, p.top_k, p.top_p, 70 + i, d)
                for i, p in enumerate(plain + other)]
        assert want[3] == 0
        assert draw(list(range(7)), plain + other, 3, d) == want
        assert draw([0, 1, 2, 3], plain, 1, d) == want[:4] == draw([0, 1, 2, 3], plain, 3, d)
        assert draw([4, 5, 6], other, 2, d) == want[4:] == draw([4, 5, 6], other, 3, d)
    from fllm_amd.kernels import KernelError
    with pytest.raises(KernelError, match="kinds"):
        draw([0], plain[:1], 0, 0)
    counters = type(ops)._workspaces[torch.cuda.current_device()][: 64 * 1024]
    torch.cuda.synchronize()
    assert int(counters.to(torch.int64).sum()) == 0


@pytest.mark.parametrize("vocab", [20000, 128256, 140000])
def test_sample_rows_with_a_small_top_k_share_workgroups(ops, vocab):
    """Rows with a top-k of at most 64 are cut into parts for several workgroups (vocabularies of 8,193 to 131,072
    tokens); every token is the plain sampler's, with or without the caller's hint, beside rows of other kinds: equal
    logits at the threshold (all kept), thousands of equal logits (the part hands the row back), a distribution so
    peaked that fewer than k tokens lie within the histogram's reach, -inf nearly everywhere, min-p and top-p behind
    top-k, k = 1 and k = 64, and a top-k of 65 that goes the old way."""
    from fllm_amd.sampling import SampleRequest, SamplingParams, pack_rows
    g = gen(31)
    params = [SamplingParams(temperature=0.8, top_k=50, top_p=0.9), SamplingParams(temperature=1.0, top_k=5),
              SamplingParams(temperature=1.3, top_k=64, min_p=0.05, top_p=0.7), SamplingParams(temperature=0.7, top_k=1),
              SamplingParams(temperature=1.0, top_k=40), SamplingParams(temperature=1.0, top_k=40), SamplingParams(temperature=2.0, top_k=30),
              SamplingParams(temperature=1.0, top_k=10), SamplingParams(temperature=0.9, top_k=65, top_p=0.95),
              SamplingParams(temperature=1.0), SamplingParams(temperature=0.0), SamplingParams(temperature=1.1, top_p=0.5)]
    logits = torch.randn(len(params), vocab, generator=g) * 3.0
    logits[1, 100:140] = float(logits[1].max()) + 1.0                 # forty equal largest logits and a top-k of 5: all stay
    logits[4, :] = torch.round(logits[4])                              # a few distinct values: thousands of equals in a part
    logits[5, :] = -200.0 + 0.001 * torch.randn(vocab, generator=g)    # peaked: three tokens far above everything else
    logits[5, [7, vocab // 2, vocab - 1]] = torch.tensor([0.0, -0.5, -1.0])
    logits[6, :] = float("-inf")
    logits[6, [3, 9000, vocab - 2]] = torch.tensor([1.0, 0.5, 2.0])
    logits[7, ::3] = float("nan")

    def draw(kinds, d):
        reqs = [SampleRequest(p, seed=900 + i, draw=d) for i, p in enumerate(params)]
        out = torch.full((len(params),), -1, dtype=torch.int32, device=DEV)
        ops.sample(logits.to(DEV), torch.empty(len(params), vocab, device=DEV), pack_rows(reqs).to(DEV), out, kinds)
        return out.cpu().tolist()

    for d in range(4):
        want = [plain_llama.device_sample(logits[i].numpy(), p.temperature, p.top_k, p.top_p, 900 + i, d, p.min_p) for i, p in enumerate(params)]
        assert draw(7, d) == want, d
        assert draw(3, d) == want, d                # without the hint the single workgroup does it
    assert {draw(7, d)[1] for d in range(12)} <= set(range(100, 140)) and len({draw(7, d)[1] for d in range(12)}) > 3
    counters = type(ops)._workspaces[torch.cuda.current_device()][: 64 * 1024]
    torch.cuda.synchronize()
    assert int(counters.to(torch.int64).sum()) == 0


def test_adjust_logits(ops):
    """Penalties, biases, blocked and allowed ids on rows of logits against the plain functions: a row with everything, a row
    whose newest token is on the device only and already in its list (it counts once more), one whose newest token
    is new to the list, a row left alone, ids outside the vocabulary ignored; an allow list (every other token goes,
    at a vocabulary that is no multiple of the workgroup); pairs that block a token if the newest token, on the
    device, is a given one, in a row without penalties and in one whose penalties look at no token."""
    from fllm_amd.sampling import SamplingParams
    from fllm_amd.sampling.adjust import AdjustRow, pack
    g = gen(41)
    vocab = 1000
    logits = torch.randn(8, vocab, generator=g) * 3.0
    logits[0, 17] = float("nan")
    last_tokens = torch.tensor([5, 123, 999], dtype=torch.int32)
    full = SamplingParams(repetition_penalty=1.7, presence_penalty=0.3, frequency_penalty=0.2, logit_bias=((3, 2.5), (17, 1.0), (4000, 9.0)))
    allowed = (0, 5, 6, 400, 998, 999, 4000)
    rows = [AdjustRow(full, {5: 2, 17: 1, 900: 4, 4000: 1, 44: 3}, blocked=(1, 2, 4000)),
            AdjustRow(SamplingParams(frequency_penalty=0.5), {123: 2, 7: 1}, last_row=1),
            AdjustRow(SamplingParams(repetition_penalty=0.5), {7: 1}, last_row=2),
            None,
            AdjustRow(SamplingParams(min_tokens=3), {}, blocked=(0, 999)),
            AdjustRow(SamplingParams(allowed_token_ids=allowed, presence_penalty=1.0), {5: 1, 7: 2}, blocked=(6,), allowed=allowed),
            AdjustRow(SamplingParams(bad_word_ids=((1, 2),)), {}, last_row=1, pairs=((123, 40), (124, 41), (123, 4000))),
            AdjustRow(SamplingParams(repetition_penalty=3.0, repeat_last_n=0), {}, last_row=0, pairs=((5, 50), (6, 51)))]
    packed, sections = pack(rows)
    got = ops.adjust_logits(logits.clone().to(DEV), packed.to(DEV), sections, last_tokens.to(DEV)).cpu()
    histories = [[5, 5, 17, 900, 900, 900, 900, 4000, 44, 44, 44], [123, 123, 7, 123], [7, 999], [], [], [5, 7, 7], [], []]
    also_blocked = [(), (), (), (), (), (), (40,), (50,)]
    for r, row in enumerate(rows):
        want = logits[r].numpy()
        if row is not None:
            p = row.params
            want = plain_llama.apply_penalties(want, histories[r], p.repetition_penalty, p.presence_penalty, p.frequency_penalty, -1,
                                               p.logit_bias)
            want[[t for t in row.blocked + also_blocked[r] if t < vocab]] = -np.inf
            want = plain_llama.apply_generation_controls(want, 0, 0, (), (), row.allowed)
        assert np.array_equal(got[r].numpy(), want, equal_nan=True), r
    assert torch.equal(got[3], logits[3])
    assert int(torch.isfinite(got[5]).sum()) == 5 and torch.equal(got[7, :50], logits[7, :50])


@pytest.mark.parametrize("vocab,top", [(300, 0), (1000, 5), (128256, 20), (7, 7)])
def test_logprobs(ops, vocab, top):
    """Log-probabilities of the chosen token and the likeliest ones against the plain function: equal values come in
    token order, -inf entries have no probability, a row with a NaN has no distribution, rows that were not asked for
    are not touched, and only the wanted rows are read."""
    g = gen(60 + top)
    rows = 6
    logits = torch.randn(rows, vocab, generator=g) * 5.0
    best = int(logits[1].argmax())
    logits[1, (best + 3) % vocab] = logits[1, best]           # two equal largest values
    logits[1, vocab - 1] = logits[1, best]
    logits[2, ::2] = -float("inf")
    logits[3, 5 % vocab] = float("nan")
    logits[4] = 1000.0 + torch.arange(vocab) % 3             # only three distinct values, far from zero
    logits[5, 1:] = -float("inf")                             # one token has it all
    tokens = torch.tensor([int(logits[r].nan_to_num(-1e30).argmax()) for r in range(rows)], dtype=torch.int32)
    tokens[0] = vocab - 1                                      # an unlikely token was drawn
    tokens[2] = 0                                              # one that cannot be: -inf
    wanted = [5, 0, 1, 2, 3, 4][:rows - (1 if top == 0 else 0)]
    values = torch.full((len(wanted), 1 + top), 7.0, device=DEV)
    ids = torch.full((len(wanted), 1 + top), 7, dtype=torch.int32, device=DEV)
    ops.logprobs(logits.to(DEV), torch.tensor(wanted, dtype=torch.int32, device=DEV), tokens.to(DEV), top, values, ids)
    values, ids = values.cpu(), ids.cpu()
    for w, r in enumerate(wanted):
        want = plain_llama.raw_logprobs(logits[r].numpy(), int(tokens[r]), top)
        assert int(ids[w, 0]) == int(tokens[r])
        if want is None:
            assert r == 3 and bool(torch.isnan(values[w]).all()) and ids[w, 1:].tolist() == [-1] * top
            continue
        chosen, alternatives = want
        assert ids[w, 1:].tolist() == [i for i, _ in alternatives], (r, ids[w].tolist())
        got = np.array([float(values[w, 0])] + values[w, 1:].tolist())
        expected = np.array([chosen] + [v for _, v in alternatives])
        finite = np.isfinite(expected)
        assert np.array_equal(got[~finite], expected[~finite])
        if finite.any():
            assert np.abs(got[finite] - expected[finite]).max() <= 2e-6 * max(1.0, np.abs(expected[finite]).max()) + 2e-6, r
    with pytest.raises(Exception, match="at most"):
        ops.logprobs(logits.to(DEV), torch.tensor([0], dtype=torch.int32, device=DEV), tokens.to(DEV), 21,
                     torch.empty(1, 22, device=DEV), torch.empty(1, 22, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("vocab,top", [(300, 3), (1000, 5), (128256, 20), (7, 7)])
def test_logprobs_of_the_distribution_a_token_was_drawn_from(ops, vocab, top):
    """`logprobs_processed` against the plain function: greedy rows are point masses, sampled rows the softmax of
    logits / T over what top-k, min-p and top-p leave (ties at a threshold kept, as the sampler keeps them); a token
    outside the support has -inf, fewer survivors than alternatives leave the rest empty, and the token the sampler
    draws from the same records lies inside the support."""
    from fllm_amd.sampling import SampleRequest, SamplingParams, pack_rows
    g = gen(80 + top)
    settings = [dict(temperature=0.0), dict(temperature=0.8), dict(temperature=1.3, top_k=4), dict(temperature=0.7, top_p=0.6),
                dict(temperature=1.0, top_k=50, top_p=0.9, min_p=0.02), dict(temperature=0.9, min_p=0.1), dict(temperature=0.5, top_k=2),
                dict(temperature=1.1, top_k=3)]
    rows = len(settings)
    logits = torch.randn(rows, vocab, generator=g) * 3.0
    logits[2, ::3] = -float("inf")
    best = int(logits[7].argmax())
    logits[7, (best + 1) % vocab] = logits[7, best]            # equal values at the top: top-k keeps its ties
    logits[7, (best + 2) % vocab] = logits[7, best]
    logits[7, (best + 3) % vocab] = logits[7, best]
    requests = [SampleRequest(SamplingParams(**s), seed=11 + r, draw=r) for r, s in enumerate(settings)]
    params = pack_rows(requests).to(DEV)
    drawn = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), torch.empty(rows, vocab, device=DEV), params, drawn)
    tokens = drawn.cpu().clone()
    tokens[6] = int(torch.argsort(logits[6], descending=True)[min(5, vocab - 1)])      # a token top-k 2 leaves out
    wanted = [3, 0, 1, 2, 4, 5, 6, 7]
    values = torch.full((len(wanted), 1 + top), 7.0, device=DEV)
    ids = torch.full((len(wanted), 1 + top), 7, dtype=torch.int32, device=DEV)
    ops.logprobs_processed(logits.to(DEV), torch.tensor(wanted, dtype=torch.int32, device=DEV), tokens.to(DEV), params, top, values, ids)
    values, ids = values.cpu(), ids.cpu()
    for w, r in enumerate(wanted):
        s = settings[r]
        chosen, alternatives = plain_llama.processed_logprobs(logits[r].numpy(), int(tokens[r]), top, s["temperature"], s.get("top_k", 0),
                                                              s.get("top_p", 1.0), s.get("min_p", 0.0))
        assert int(ids[w, 0]) == int(tokens[r])
        assert ids[w, 1:].tolist() == [i for i, _ in alternatives] + [-1] * (top - len(alternatives)), (r, ids[w].tolist())
        got = np.array([float(values[w, 0])] + values[w, 1:1 + len(alternatives)].tolist())
        expected = np.array([chosen] + [v for _, v in alternatives])
        finite = np.isfinite(expected)
        assert np.array_equal(got[~finite], expected[~finite]), r
        assert np.abs(got[finite] - expected[finite]).max() <= 2e-5, r
        assert bool(torch.isnan(values[w, 1 + len(alternatives):]).all())
        if r != 6:
            assert math.isfinite(float(values[w, 0])), f"row {r}: the sampler drew a token outside the support"
    assert float(values[wanted.index(6), 0]) == -math.inf and float(values[wanted.index(0), 0]) == 0.0
    assert len([i for i in ids[wanted.index(7), 1:].tolist() if i >= 0]) == min(top, 4)       # four equal largest values survive top-k 3


def test_sample_depends_only_on_seed_draw_and_logits(ops):
    from fllm_amd.sampling import SampleRequest, SamplingParams, pack_rows
    g = gen(18)
    vocab = 128256
    logits = torch.randn(4, vocab, generator=g)
    p = SamplingParams(temperature=0.9, top_k=40, top_p=0.95)
    reqs = [SampleRequest(p, seed=5, draw=d) for d in (0, 1, 2, 1)]
    lg = logits.clone()
    lg[3] = lg[1]
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    ops.sample(lg.to(DEV), torch.empty(4, vocab, device=DEV), pack_rows(reqs).to(DEV), out)
    alone = torch.empty(1, dtype=torch.int32, device=DEV)
    ops.sample(lg[1:2].to(DEV), torch.empty(1, vocab, device=DEV), pack_rows(reqs[1:2]).to(DEV), alone)
    assert int(out[1]) == int(out[3]) == int(alone[0])
    top40 = set(torch.topk(lg[0], 40).indices.tolist())
    assert int(out[0]) in top40


def test_a_second_stream_is_refused(ops):
    """Kernels of a device meet in its workspace: launches on another stream could overlap with those on the first and
    are refused; a stream that captures a graph is let through (the engine's decode graphs are captured that way)."""
    from fllm_amd.kernels import KernelError
    x = torch.randn(4, 64, device=DEV)
    w = torch.ones(64, device=DEV)
    out = torch.empty(4, 64, device=DEV)
    ops.rmsnorm(x, w, 1e-5, out)
    other = torch.cuda.Stream()
    with torch.cuda.stream(other):
        with pytest.raises(KernelError, match="one stream"):
            ops.rmsnorm(x, w, 1e-5, out)
    torch.cuda.synchronize()
    want = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.rmsnorm(x, w, 1e-5, out)
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want)
