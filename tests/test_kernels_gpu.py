"""Each HIP kernel alone against a plain PyTorch reference of the same
operation, at sizes other than the engine's, in float32 and in bfloat16."""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def K():
    from lockstep_amd.ops import kernels

    return kernels()


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


TOL = {torch.float32: 2e-5, torch.bfloat16: 1.5e-2}


# -- matrix product ------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 16, 32), (1, 1000, 96), (5, 48, 200), (16, 100, 64), (17, 33, 72),
                                   (64, 256, 1024), (65, 130, 260), (37, 3072, 1024), (200, 96, 4100),
                                   (130, 1000, 8), (3, 40, 12),
                                   # 128 x 128 tiles with rows, columns and K that end inside a tile (operand
                                   # loads from clamped addresses), and the same with K not 16-byte aligned
                                   (2050, 2100, 264), (2050, 2100, 260),
                                   # an odd K: no operand row is 16-byte aligned, in either precision
                                   (200, 90, 101), (9, 50, 37)])
def test_gemm_matches_linear(dtype, m, n, k):
    from lockstep_amd.ops import STORE, STORE_F32, ADD_F32

    g = torch.Generator().manual_seed(m * 1000 + n + k)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = torch.randn(n, k, generator=g).to(dtype)
    want = x.double() @ w.double().T
    xd, wd = x.cuda(), w.cuda()
    out = torch.empty(m, n, dtype=dtype, device="cuda")
    K().gemm(xd, wd, out, STORE)
    assert rel_err(out, want) < TOL[dtype]
    out32 = torch.empty(m, n, dtype=torch.float32, device="cuda")
    K().gemm(xd, wd, out32, STORE_F32)
    assert rel_err(out32, want) < (2e-5 if dtype is torch.float32 else 2e-5 + 0)  # float accumulate: tight in both
    base = torch.randn(m, n, generator=g)
    acc = base.cuda()
    K().gemm(xd, wd, acc, ADD_F32)
    assert rel_err(acc, base.double() + want) < 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_row_does_not_depend_on_the_batch(dtype):
    """Row i alone, in a 16-row batch, in a 64-row batch and in a 300-row batch:
    same bits (the skinny and the tiled kernel share one summation order)."""
    from lockstep_amd.ops import STORE_F32

    g = torch.Generator().manual_seed(7)
    # the last shape has so many columns that 17 to 64 rows already take the tiled kernel
    for k, n in ((1024, 272), (3072, 96), (200, 130), (5000, 64), (96, 32768 + 40)):
        x = torch.randn(300, k, generator=g).to(dtype).cuda()
        w = torch.randn(n, k, generator=g).to(dtype).cuda()
        full = torch.empty(300, n, dtype=torch.float32, device="cuda")
        K().gemm(x, w, full, STORE_F32)
        for rows in (1, 16, 17, 64, 65, 128):
            part = torch.empty(rows, n, dtype=torch.float32, device="cuda")
            K().gemm(x[:rows], w, part, STORE_F32)
            assert torch.equal(part, full[:rows]), f"rows={rows} k={k} n={n}"
        for i in (0, 1, 17, 63, 64, 299):
            one = torch.empty(1, n, dtype=torch.float32, device="cuda")
            K().gemm(x[i:i + 1], w, one, STORE_F32)
            assert torch.equal(one[0], full[i]), f"row {i} k={k} n={n}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k,n", [(4096, 4096 + 24), (1000, 16384 + 24), (5120, 4096 + 104), (260, 32768 + 40),
                                 # slices of 512 and some 7,000 columns: from 32 rows on tiles of 64 x 32 outputs
                                 (5120, 7168 + 24), (1000, 6144 + 8),
                                 (2048, 8192 + 8), (96, 65536 + 48),
                                 # K of 5,120 over so many columns that tiles of 64 x 128 give every CU one
                                 (5120, 36864 + 72)])
def test_gemm_with_few_rows_and_many_columns_has_the_same_bits(dtype, k, n):
    """With up to 64 rows and more column blocks than the GPU holds workgroups, a workgroup walks
    several column blocks with its rows of X in registers (the streaming kernel; beyond 32 rows two
    groups of workgroups take 32 rows each).  Every row has the bits it has in a large batch, with
    every epilogue; a row of the sums equals the double precision product."""
    from lockstep_amd.ops import ADD_F32, STORE, STORE_F32

    g = torch.Generator().manual_seed(k + n)
    x = torch.randn(200, k, generator=g).to(dtype).cuda()
    w = (torch.randn(n, k, generator=g) * 0.1).to(dtype).cuda()
    full = torch.empty(200, n, dtype=torch.float32, device="cuda")
    K().gemm(x, w, full, STORE_F32)
    want = x[:3].double().cpu() @ w.double().cpu().T
    assert rel_err(full[:3], want) < 2e-5
    base = torch.randn(64, n, generator=g).cuda()
    for rows in (1, 8, 16, 17, 32, 33, 50, 64):
        part = torch.empty(rows, n, dtype=torch.float32, device="cuda")
        K().gemm(x[:rows], w, part, STORE_F32)
        assert torch.equal(part, full[:rows]), f"rows={rows}"
        stored = torch.empty(rows, n, dtype=dtype, device="cuda")
        K().gemm(x[:rows], w, stored, STORE)
        assert torch.equal(stored, full[:rows].to(dtype)), f"rows={rows}, stored in {dtype}"
        acc = base[:rows].clone()
        K().gemm(x[:rows], w, acc, ADD_F32)
        assert torch.equal(acc, base[:rows] + full[:rows]), f"rows={rows}, added"
    one = torch.empty(1, n, dtype=torch.float32, device="cuda")
    K().gemm(x[31:32], w, one, STORE_F32)
    assert torch.equal(one[0], full[31])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [264, 1088])
def test_gemm_with_many_rows_and_columns_has_the_bits_of_few_rows(dtype, k):
    """2,050 rows by 3,740 columns: 17 x 15 tiles of 128 x 256 outputs fill one round of 256 CUs, so
    bfloat16 takes the workgroups of eight waves; rows, columns and (with 264) K end inside a tile.
    Every epilogue; rows from all over the product have the bits they have in a product of 40 rows,
    which the skinny kernel computes."""
    from lockstep_amd.ops import ADD_F32, STORE, STORE_F32, SWIGLU, interleave_gate_up

    g = torch.Generator().manual_seed(k)
    m, n = 2050, 3740
    x = torch.randn(m, k, generator=g).to(dtype).cuda()
    w = (torch.randn(n, k, generator=g) * 0.1).to(dtype).cuda()
    full = torch.empty(m, n, dtype=torch.float32, device="cuda")
    K().gemm(x, w, full, STORE_F32)
    want = x[-3:].double().cpu() @ w.double().cpu().T
    assert rel_err(full[-3:], want) < 2e-5
    stored = torch.empty(m, n, dtype=dtype, device="cuda")
    K().gemm(x, w, stored, STORE)
    assert torch.equal(stored, full.to(dtype))
    base = torch.randn(m, n, generator=g).cuda()
    acc = base.clone()
    K().gemm(x, w, acc, ADD_F32)
    assert torch.equal(acc, base + full)
    inter = n // 2
    wi = interleave_gate_up(w[:inter].cpu(), w[inter:].cpu()).cuda()
    gated = torch.empty(m, inter, dtype=dtype, device="cuda")
    K().gemm(x, wi, gated, SWIGLU)
    for first in (0, 100, 1000, 2010):
        rows = slice(first, first + 40)
        part = torch.empty(40, n, dtype=torch.float32, device="cuda")
        K().gemm(x[rows], w, part, STORE_F32)
        assert torch.equal(part, full[rows]), f"rows from {first}"
        part = torch.empty(40, inter, dtype=dtype, device="cuda")
        K().gemm(x[rows], wi, part, SWIGLU)
        assert torch.equal(part, gated[rows]), f"rows from {first}, SwiGLU"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter,k", [(4096 + 40, 4096), (16384 + 72, 1024), (25600, 5120)])
def test_swiglu_with_few_rows_and_many_columns_has_the_same_bits(dtype, inter, k):
    from lockstep_amd.ops import SWIGLU, interleave_gate_up

    g = torch.Generator().manual_seed(inter + k)
    x = torch.randn(150, k, generator=g).to(dtype).cuda()
    gate = (torch.randn(inter, k, generator=g) * 0.05).to(dtype)
    up = (torch.randn(inter, k, generator=g) * 0.05).to(dtype)
    w = interleave_gate_up(gate, up).cuda()
    full = torch.empty(150, inter, dtype=dtype, device="cuda")
    K().gemm(x, w, full, SWIGLU)
    want = torch.nn.functional.silu(x[:2].double().cpu() @ gate.double().T) * (x[:2].double().cpu() @ up.double().T)
    assert rel_err(full[:2], want) < TOL[dtype]
    for rows in (1, 8, 16, 20, 32, 40, 64):
        part = torch.empty(rows, inter, dtype=dtype, device="cuda")
        K().gemm(x[:rows], w, part, SWIGLU)
        assert torch.equal(part, full[:rows]), f"rows={rows}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [1024, 4096, 5120])
def test_the_full_vocabulary_head_against_double_precision(dtype, k):
    """151,936 columns (the streaming kernel for few rows, tiles of 64 x 128 up to 64 rows, large tiles
    beyond) at 1, 8, 64 and 200 rows: every row equals the double-precision product and has the
    same bits at every number of rows."""
    from lockstep_amd.ops import STORE_F32

    vocab = 151936
    g = torch.Generator(device="cuda").manual_seed(k)
    x = torch.randn(200, k, generator=g, device="cuda").to(dtype)
    w = (torch.randn(vocab, k, generator=g, device="cuda") * 0.05).to(dtype)
    want = torch.cat([x.double() @ w[lo:lo + 16384].double().T for lo in range(0, vocab, 16384)], dim=1)
    full = None
    for rows in (200, 1, 8, 64):
        out = torch.full((rows, vocab), float("nan"), device="cuda")
        K().gemm(x[:rows], w, out, STORE_F32)
        assert rel_err(out, want[:rows]) < 2e-5, rows
        if full is None:
            full = out
        assert torch.equal(out, full[:rows]), rows
    del w, want, full
    torch.cuda.empty_cache()


@pytest.mark.parametrize("vocab", [7, 1000, 4099, 151936])
def test_the_sampling_kernel_picks_the_host_samplers_token(vocab):
    """Temperature and nucleus sampling on the device against the host procedure (float64, sorted): the same
    token for every row, with spread-out and with quantised logits (many equal values: the order among
    equals is the order of the ids), small and large nuclei, several temperatures; twice the same."""
    from lockstep_amd.sampling import philox
    from lockstep_amd.sampling.sampler import top_p as host_top_p

    n = 48 if vocab < 100000 else 12
    g = torch.Generator().manual_seed(vocab)
    logits = torch.randn(n + 3, vocab, generator=g) * (0.5 + 3 * torch.rand(n + 3, 1, generator=g))
    logits[::5] = torch.round(logits[::5] * 2) / 2
    logits[1, : vocab // 2] = logits[1, 0]                          # half of the row is one value
    rows = torch.randperm(n + 3, generator=g)[:n].to(torch.int32)
    temperature = [[0.3, 0.8, 1.0, 1.7][i % 4] for i in range(n)]
    nucleus = [[1.0, 0.9, 0.5, 0.05, 0.999, 0.0][i % 6] for i in range(n)]
    seed = 7 + (1 << 40)                          # both halves of the key in use
    # the host procedure with the same seed, uid and position (positions beyond 32 bits too)
    positions = [i if i % 7 else (5 << 32) + i for i in range(n)]
    want = [host_top_p(logits[int(rows[i])], seed, "kernel", positions[i], nucleus[i], temperature[i]) for i in range(n)]
    dev = logits.cuda()
    requests = [(int(rows[i]), temperature[i], nucleus[i], seed ^ philox.uid_key("kernel"), positions[i]) for i in range(n)]
    out = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    K().sample_top_p(dev, requests, out)
    assert out.cpu().tolist() == want
    again = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    K().sample_top_p(dev, requests, again)
    assert torch.equal(out, again)
    assert len(set(want)) > 1


def sample_among(kernels, dev, requests, n_rows: int, order_seed: int):
    """The tokens of ``requests`` when they are sampled in one call of ``n_rows`` rows (the others
    being further draws from the same logits rows), in a shuffled order."""
    base = len(requests)
    extra = [(i % base, 0.5 + (i % 7) / 4, [1.0, 0.8][i % 2], 900 + i, 50000 + i) for i in range(max(0, n_rows - base))]
    every = list(requests[:n_rows]) + extra
    order = torch.randperm(len(every), generator=torch.Generator().manual_seed(order_seed)).tolist()
    out = torch.full((len(every),), -1, dtype=torch.int32, device="cuda")
    kernels.sample_top_p(dev, [every[j] for j in order], out)
    picked = out.cpu().tolist()
    tokens = [None] * len(every)
    for place, j in enumerate(order):
        tokens[j] = picked[place]
    return tokens[:min(n_rows, base)]


@pytest.mark.parametrize("vocab", [1000, 151936])
def test_a_sampled_row_gets_the_same_token_beside_any_number_of_other_rows(vocab):
    """The same logits rows sampled alone and in calls of 24, 33, 64 and 200 rows: the same tokens.
    Half of the rows are spread-out logits with random nuclei; the other half are made so that a
    change in the order of any sum would show (``sampling_rows_on_boundaries``: the positive
    control of this test runs them against a sampler whose cut depends on the rows of the call)."""
    from helpers import sampling_rows_on_boundaries
    from lockstep_amd.sampling import philox

    g = torch.Generator().manual_seed(vocab + 1)
    spread = torch.randn(12, vocab, generator=g) * 2.0
    spread[::2] = torch.round(spread[::2] * 4) / 4
    spread[3, : vocab // 3] = 1.25
    spread[5] = 0.0                                                 # one value only: the draw counts ties off
    sharp, on_boundaries = sampling_rows_on_boundaries(vocab, rows=12)
    dev = torch.cat([spread, sharp]).cuda()
    key = philox.uid_key("same-row")
    requests = [(i, [0.7, 1.0, 1.9][i % 3], [1.0, 0.9, 0.3, 0.999][i % 4], (11 + i) ^ key, 1000 + 17 * i) for i in range(12)]
    requests += [(12 + row, t, p, k, pos) for row, t, p, k, pos in on_boundaries]
    alone = []
    for request in requests:                                        # every request in a call of its own
        out = torch.full((1,), -1, dtype=torch.int32, device="cuda")
        K().sample_top_p(dev, [request], out)
        alone.append(int(out.item()))
    assert all(0 <= t < vocab for t in alone)
    for n_rows in (len(requests), 33, 64, 200):
        assert sample_among(K(), dev, requests, n_rows, n_rows) == alone, f"{n_rows} rows in the call"


def test_the_sampler_takes_greedy_and_drawn_rows_of_one_step_together():
    from lockstep_amd.sampling import Sampler
    from lockstep_amd.sampling.sampler import top_p as host_top_p

    class Row:
        def __init__(self, uid, seed, temperature, nucleus, total):
            self.uid, self.seed, self.temperature, self.top_p, self._total = uid, seed, temperature, nucleus, total

        def total_tokens(self):
            return self._total

    g = torch.Generator().manual_seed(3)
    logits = torch.randn(6, 5003, generator=g) * 2
    requests = [Row("a", 1, 0.0, 1.0, 5), Row("b", 2, 0.7, 0.9, 9), Row("c", 3, 0.0, 1.0, 2), Row("d", 4, 1.3, 1.0, 40),
                Row("e", 5, 0.2, 0.3, 7), Row("f", 6, 1.0, 0.95, 1)]
    want = [host_top_p(logits[i], r.seed, r.uid, r.total_tokens() - 1, r.top_p, r.temperature) for i, r in enumerate(requests)]
    assert Sampler(K()).sample(logits.cuda(), requests) == want


def test_gemm_refuses_mismatched_operands():
    from lockstep_amd.ops import KernelError

    x = torch.zeros(4, 32, device="cuda")
    w = torch.zeros(8, 48, device="cuda")
    with pytest.raises(KernelError):
        K().gemm(x, w, torch.zeros(4, 8, device="cuda"))


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("activation", ["none", "silu", "gelu_tanh", "gelu", "relu"])
@pytest.mark.parametrize("rows,width", [(1, 40), (7, 1000), (70, 3072)])
def test_bias_and_activation_pass_against_torch(out_dtype, activation, rows, width):
    """``act(x + bias)`` and its gated form ``act(gate + b) * (up + b)``, with and without a bias, also in place."""
    g = torch.Generator().manual_seed(rows + width)
    acts = {"none": lambda v: v, "silu": torch.nn.functional.silu, "relu": torch.relu,
            "gelu": torch.nn.functional.gelu, "gelu_tanh": lambda v: torch.nn.functional.gelu(v, approximate="tanh")}
    tol = 2e-6 if out_dtype is torch.float32 else 5e-3
    for gated in (False, True):
        x = torch.randn(rows, width * (2 if gated else 1) + 8, generator=g).cuda()[:, : width * (2 if gated else 1)]
        for bias in (None, torch.randn(x.shape[1], generator=g).cuda()):
            out = torch.full((rows, width), float("nan"), dtype=out_dtype, device="cuda")
            K().bias_act(x, bias, out, activation, gated=gated)
            v = x.double() + (bias.double() if bias is not None else 0.0)
            want = acts[activation](v[:, :width]) * (v[:, width:] if gated else 1.0)
            assert rel_err(out, want) < tol, (activation, gated, bias is not None)
    x = torch.randn(rows, width, generator=g).cuda()
    bias = torch.randn(width, generator=g).cuda()
    want = acts[activation](x.double() + bias.double())
    K().bias_act(x, bias, x, activation)                        # in place
    assert rel_err(x, want) < 2e-6
    from lockstep_amd.ops import KernelError
    with pytest.raises(KernelError, match="not built"):
        K().bias_act(x, None, x, "swish7")
    with pytest.raises(KernelError, match="float32 \\["):
        K().bias_act(x, None, torch.empty(rows, width + 1, device="cuda"), "none")


# -- norm --------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width,eps", [(1, 64, 1e-6), (7, 96, 1e-5), (48, 1024, 1e-6), (3, 5120, 1e-6),
                                            (5, 100, 1e-3)])
def test_rmsnorm_matches_formula(dtype, rows, width, eps):
    g = torch.Generator().manual_seed(width)
    x = torch.randn(rows, width, generator=g) * 3
    w = 1 + 0.1 * torch.randn(width, generator=g)
    want = x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + eps) * w.double()
    out = torch.empty(rows, width, dtype=dtype, device="cuda")
    K().rmsnorm(x.cuda(), w.cuda(), out, eps)
    assert rel_err(out, want) < (1e-6 if dtype is torch.float32 else 5e-3)
    lib = torch.nn.functional.rms_norm(x, (width,), w, eps)
    assert rel_err(out, lib) < (1e-6 if dtype is torch.float32 else 5e-3)
    # selected rows, and a row alone gives the same bits as in the batch
    idx = torch.tensor([rows - 1, 0], dtype=torch.int32, device="cuda")
    sel = torch.empty(2, width, dtype=dtype, device="cuda")
    K().rmsnorm(x.cuda(), w.cuda(), sel, eps, idx)
    assert torch.equal(sel[0], out[rows - 1]) and torch.equal(sel[1], out[0])


# -- SwiGLU, embedding, arg-max --------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_matches_silu_times_up(dtype):
    g = torch.Generator().manual_seed(1)
    gu = (torch.randn(7, 2 * 300, generator=g) * 2).to(dtype)
    want = torch.nn.functional.silu(gu[:, :300].double()) * gu[:, 300:].double()
    out = torch.empty(7, 300, dtype=dtype, device="cuda")
    K().swiglu(gu.cuda(), out)
    assert rel_err(out, want) < (1e-6 if dtype is torch.float32 else 5e-3)
    zero = torch.zeros(2, 64, dtype=dtype, device="cuda")
    out0 = torch.ones(2, 32, dtype=dtype, device="cuda")
    K().swiglu(zero, out0)
    assert torch.count_nonzero(out0) == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_gathers_rows(dtype):
    table = torch.randn(1000, 96).to(dtype)
    ids = torch.tensor([0, 999, 5, 5, 731], dtype=torch.int32)
    out = torch.empty(5, 96, dtype=torch.float32, device="cuda")
    K().embed(ids.cuda(), table.cuda(), out)
    assert torch.equal(out.cpu(), table[ids.long()].float())


def test_argmax_takes_the_lowest_index_among_maxima():
    x = torch.randn(6, 151936)
    x[1, 77] = x[1, 150000] = 50.0
    x[2, :] = 1.0
    x[3, 151935] = 60.0
    out = torch.empty(6, dtype=torch.int32, device="cuda")
    K().argmax(x.cuda(), out)
    want = [int(torch.nonzero(r == r.max())[0]) for r in x]
    assert out.cpu().tolist() == want
    assert want[1] == 77 and want[2] == 0 and want[3] == 151935


def test_argmax_with_more_rows_than_the_static_scratch_holds():
    """Beyond 16,384 (row, chunk) pairs the wrapper brings a scratch buffer, and a larger call
    after a smaller one grows it; the results are those of the static path."""
    k = K()
    g = torch.Generator().manual_seed(5)
    for rows in (2100, 2900):                       # 3 chunks a row: 6,300 and 8,700 pairs, the static array
        x = torch.randn(rows, 9000, generator=g)
        x[:, 8999] = x.max(dim=1).values            # a tie with the last column: the lower index wins
        out = torch.empty(rows, dtype=torch.int32, device="cuda")
        k.argmax(x.cuda(), out)
        assert torch.equal(out.long().cpu(), (x == x.max(1, keepdim=True).values).int().argmax(1))
    for rows in (5600, 7000):                       # 16,800 and 21,000 pairs: beyond the static array, growing
        assert rows * 3 > k.ARGMAX_STATIC_PAIRS
        x = torch.randn(rows, 9000, generator=g)
        out = torch.empty(rows, dtype=torch.int32, device="cuda")
        k.argmax(x.cuda(), out)
        assert torch.equal(out.long().cpu(), x.argmax(dim=1))
    small = torch.tensor([[1.0, 5.0, 5.0, 5.0, 2.0]]).cuda()
    one = torch.empty(1, dtype=torch.int32, device="cuda")
    K().argmax(small, one)
    assert one.item() == 1
    # widths and row strides that are no multiple of four, maxima at the edges of a chunk, NaN, a view
    g = torch.Generator().manual_seed(3)
    for width in (4095, 4096, 4097, 8191, 12289, 50001):
        y = torch.randn(5, width + 3, generator=g)
        y[0, min(4095, width - 1)] = 9.0
        y[1, min(4096, width - 1)] = 9.0
        y[2, width - 1] = 9.0
        y[3, 0] = float("nan")
        y[4, :] = float("nan")
        view = y.cuda()[:, :width]
        got = torch.empty(5, dtype=torch.int32, device="cuda")
        K().argmax(view, got)
        ref = y[:, :width].clone()
        ref[ref != ref] = float("-inf")
        want = [int(torch.nonzero(r == r.max())[0]) for r in ref]
        want[4] = 0
        assert got.cpu().tolist() == want, width


# -- norm + rotation + cache write, attention ---------------------------------------------

def naive_attention(q, k, v, q_start, scale, window=None):
    """q [Tq,nq,d], k,v [Tk,nkv,d] in float64; explicit max-subtract softmax."""
    tq, nq, d = q.shape
    tk, nkv, _ = k.shape
    g = nq // nkv
    k = k.repeat_interleave(g, dim=1)
    v = v.repeat_interleave(g, dim=1)
    s = torch.einsum("qhd,khd->hqk", q, k) * scale
    qp = torch.arange(q_start, q_start + tq)[:, None]
    kp = torch.arange(tk)[None, :]
    hidden = kp > qp
    if window:
        hidden = hidden | (qp - kp >= window)
    s = s.masked_fill(hidden[None], float("-inf"))
    m = s.max(-1, keepdim=True).values
    e = (s - m).exp()
    return torch.einsum("hqk,khd->qhd", e / e.sum(-1, keepdim=True), v)


class PagedCase:
    """Lay keys and values into pages through the engine's own write kernel."""

    def __init__(self, dtype, nq, nkv, d, page_size, n_tokens, shuffle_seed=None, extra_pages=3):
        self.dtype, self.nq, self.nkv, self.d, self.ps = dtype, nq, nkv, d, page_size
        n_pages = -(-n_tokens // page_size)
        order = list(range(n_pages + extra_pages))
        if shuffle_seed is not None:
            g = torch.Generator().manual_seed(shuffle_seed)
            order = torch.randperm(n_pages + extra_pages, generator=g).tolist()
        self.table = torch.full((2, n_pages + 1), -1, dtype=torch.int32)
        self.table[1, :n_pages] = torch.tensor(order[:n_pages], dtype=torch.int32)
        self.table = self.table.cuda()
        total = n_pages + extra_pages
        self.k_pages = torch.full((total, nkv, page_size, d), float("nan"), dtype=dtype, device="cuda")
        self.v_pages = torch.full((total, nkv, d, page_size), float("nan"), dtype=dtype, device="cuda")

    def seqs(self, q_start, q_len):
        return torch.tensor([0, q_len, q_start, q_start + q_len, 1, 0, 0, 0], dtype=torch.int32).cuda()

    def write(self, qkv, q_start, q_norm=None, k_norm=None, eps=1e-6, cos=None, sin=None, rot=0):
        t = qkv.shape[0]
        tok_seq = torch.zeros(t, dtype=torch.int32, device="cuda")
        tok_pos = torch.arange(q_start, q_start + t, dtype=torch.int32, device="cuda")
        K().qk_rope_kv(qkv, t, self.nq, self.nkv, self.d, q_norm, k_norm, eps, cos, sin, rot, tok_seq, tok_pos,
                       self.seqs(q_start, t), q_start + t - 1, self.table, self.k_pages, self.v_pages, self.ps, True)

    def attend(self, qkv, q_start, scale, window=0, force_split=None, variant=0, repeat=1, span=1, pad_splits=0,
               few_rows=False):
        """``few_rows``: tell the fold that no request has more than 16 rows (it then takes the kernel that
        asks for many splits at a time).  ``span``: splits one work item walks when the request is cut (the cooperative kernel takes more
        than one and leaves a partial result for each); ``pad_splits``: lay the items out for that many
        more splits than the request has (as the fixed-shape lists of graph-replayed steps do)."""
        from lockstep_amd.ops import kernels

        t = qkv.shape[0]
        tile, split = kernels().attention_geometry(self.d)
        g = self.nq // self.nkv
        rows = t * g
        kv_len = q_start + t
        lo = max(0, q_start - window + 1) if window else 0
        split_lo = lo // split
        n_splits = (kv_len - 1) // split + 1 - split_lo
        use_split = (rows <= 64 and n_splits > 1) if force_split is None else force_split
        items, combine, part_rows = [], [], 0
        br = kernels().attention_block_rows(self.d, variant)       # rows of a work item's row block
        if use_split:
            n_splits += pad_splits
            part_rows = self.nkv * rows * n_splits
            for b in range(-(-rows // br)):
                for s in range(split_lo, split_lo + n_splits, span):
                    items += [0, b, s, min(s + span, split_lo + n_splits), 0, n_splits, split_lo, 0]
            for b in range(-(-rows // 64)):
                combine += [0, b, 0, n_splits]
        else:
            for b in range(-(-rows // br)):
                first = q_start + (b * br) // g
                last = q_start + min(b * br + br - 1, rows - 1) // g
                begin = (max(0, first - window + 1) // split) if window else 0
                items += [0, b, begin, last // split + 1, -1, 0, 0, 0]
        from lockstep_amd.ops import pack_attention_items, pack_combine_items

        items = items * repeat      # the same work many times over (same values to the same places): a full GPU
        seq_row = self.seqs(q_start, t).cpu().numpy()
        n_items = len(items) // 8
        items_t = torch.from_numpy(pack_attention_items(items, seq_row)).to(torch.int32).cuda()
        out = torch.full((t, self.nq * self.d), float("nan"), dtype=self.dtype, device="cuda")
        part_acc = torch.full((max(part_rows, 1), self.d), float("nan"), dtype=torch.float32, device="cuda")
        part_ml = torch.full((max(part_rows, 1), 2), float("nan"), dtype=torch.float32, device="cuda")
        K().attention(qkv, self.nq, self.nkv, self.d, self.k_pages, self.v_pages, self.ps, self.table,
                      self.seqs(q_start, t), items_t, n_items, out, part_acc, part_ml, scale, window,
                      variant, rows, spans=span > 1)
        if combine:
            comb = torch.from_numpy(pack_combine_items(combine, seq_row)).to(torch.int32).cuda()
            K().attention_combine(self.d, self.seqs(q_start, t), comb, len(combine) // 4, self.nq, self.nkv,
                                  part_acc, part_ml, out, max_rows=rows if few_rows else 0)
        return out.view(t, self.nq, self.d)


def rand_qkv(t, nq, nkv, d, dtype, seed, sharp=None):
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn(t, (nq + 2 * nkv) * d, generator=g)
    if sharp is not None:
        # make one far key stand out for the last query: a fault that drops it shows
        key_pos, = sharp
        q = qkv[:, : nq * d].view(t, nq, d)
        k = qkv[:, nq * d:(nq + nkv) * d].view(t, nkv, d)
        k[key_pos] = q[-1].view(nkv, nq // nkv, d)[:, 0] * 2.0
    return qkv.to(dtype)


def split_qkv(qkv, nq, nkv, d):
    t = qkv.shape[0]
    q = qkv[:, : nq * d].reshape(t, nq, d)
    k = qkv[:, nq * d:(nq + nkv) * d].reshape(t, nkv, d)
    v = qkv[:, (nq + nkv) * d:].reshape(t, nkv, d)
    return q, k, v


ATT_TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,ps", [(16, 8, 128, 16), (4, 4, 16, 8), (8, 1, 64, 32), (6, 2, 48, 16),
                                         (32, 4, 80, 64), (2, 2, 256, 128), (64, 8, 128, 16)])
@pytest.mark.parametrize("kv_len", [1, 5, 64, 129, 257, 600])
def test_prefill_attention_matches_naive(dtype, nq, nkv, d, ps, kv_len):
    qkv = rand_qkv(kv_len, nq, nkv, d, dtype, seed=kv_len + d)
    case = PagedCase(dtype, nq, nkv, d, ps, kv_len, shuffle_seed=3)
    dev = qkv.cuda()
    case.write(dev, 0)
    out = case.attend(dev, 0, d ** -0.5)
    q, k, v = split_qkv(qkv.double(), nq, nkv, d)
    want = naive_attention(q, k, v, 0, d ** -0.5)
    assert not torch.isnan(out).any()
    assert rel_err(out, want) < ATT_TOL[dtype]
    # the kernel that loads straight from global memory gives the same bits as the LDS-staged one
    assert torch.equal(case.attend(dev, 0, d ** -0.5, variant=1), out)
    if K().wide_supported(d, dtype, ps):
        assert torch.equal(case.attend(dev, 0, d ** -0.5, variant=4), out), "wide kernel"
        assert torch.equal(case.attend(dev, 0, d ** -0.5, variant=5), out), "wide kernel, row blocks of 64"
    if kv_len == 1:
        assert torch.equal(out.cpu().float()[0], v.float()[0].repeat_interleave(nq // nkv, dim=0))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,ps", [(4, 2, 128, 16), (2, 1, 64, 8), (8, 4, 32, 64)])
def test_attention_over_more_keys_than_one_window_of_page_ids(dtype, nq, nkv, d, ps):
    """A workgroup of the streaming kernels holds the page ids of 32 tiles (4,096 keys) at a time.
    Contexts beyond that: a prompt in one step, late portions and decoded tokens, each walking all
    splits in one workgroup or cut into splits and combined; same bits in every kernel, and the
    32-bit result against the naive formula.  One far key is made to stand out."""
    n = 4096 * 2 + 300
    qkv = rand_qkv(n, nq, nkv, d, dtype, seed=n + d, sharp=(37,))
    case = PagedCase(dtype, nq, nkv, d, ps, n, shuffle_seed=5)
    dev = qkv.cuda()
    case.write(dev, 0)
    full = case.attend(dev, 0, d ** -0.5)                                  # staged or direct kernel, row blocks of 64
    q, k, v = split_qkv(qkv.double(), nq, nkv, d)
    tail = slice(n - 40, n)
    want = naive_attention(q[tail], k, v, n - 40, d ** -0.5)
    assert rel_err(full[tail], want) < ATT_TOL[dtype]
    if K().wide_supported(d, dtype, ps):
        for variant in (4, 5):
            assert torch.equal(case.attend(dev, 0, d ** -0.5, variant=variant), full), f"wide kernel {variant}"
            late = case.attend(dev[n - 200:], n - 200, d ** -0.5, variant=variant)
            assert torch.equal(late, full[n - 200:]), f"late portion, wide kernel {variant}"
    if K().coop_supported(d, dtype, ps):
        for p in (4095, 4096, 4100, 8191, 8192, n - 1):
            for split in (False, True):
                one = case.attend(dev[p:p + 1], p, d ** -0.5, variant=3, force_split=split)
                assert torch.equal(one, full[p:p + 1]), f"decoded token at {p}, split={split}"
        # with two workgroups a CU the kernel works with one buffer, refilled half by half
        crowd = case.attend(dev[n - 1:], n - 1, d ** -0.5, variant=3, force_split=False, repeat=-(-600 // nkv))
        assert torch.equal(crowd, full[n - 1:]), "decoded token, crowded launch"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,ps", [(16, 8, 128, 16), (6, 3, 32, 8), (8, 1, 64, 16)])
def test_attention_row_is_the_same_alone_in_a_portion_and_in_the_whole_prompt(dtype, nq, nkv, d, ps):
    """A query row alone (decode, split mode), in a portion, and in a whole prefill: same bits;
    also under a shuffled block table."""
    kv_len = 700
    qkv = rand_qkv(kv_len, nq, nkv, d, dtype, seed=11, sharp=(3,)).cuda()
    whole = PagedCase(dtype, nq, nkv, d, ps, kv_len)
    whole.write(qkv, 0)
    full = whole.attend(qkv, 0, d ** -0.5)
    shuffled = PagedCase(dtype, nq, nkv, d, ps, kv_len, shuffle_seed=99)
    shuffled.write(qkv, 0)
    assert torch.equal(shuffled.attend(qkv, 0, d ** -0.5), full)
    for p in (0, 1, 15, 16, 17, 127, 128, 255, 256, 257, 511, 512, 699):
        alone = whole.attend(qkv[p:p + 1], p, d ** -0.5)
        assert torch.equal(alone[0], full[p]), f"row {p} alone"
        alone = whole.attend(qkv[p:p + 1], p, d ** -0.5, variant=1)
        assert torch.equal(alone[0], full[p]), f"row {p} alone, loaded directly"
        if K().coop_supported(d, dtype, ps):
            for split in (True, False):
                alone = whole.attend(qkv[p:p + 1], p, d ** -0.5, variant=3, force_split=split)
                assert torch.equal(alone[0], full[p]), f"row {p} alone, cooperative kernel, split={split}"
        both = whole.attend(qkv[p:p + 1], p, d ** -0.5, force_split=False)
        assert torch.equal(both[0], full[p]), f"row {p} alone, direct"
    for lo, hi in ((250, 262), (0, 3), (500, 700), (255, 257), (690, 700)):
        part = whole.attend(qkv[lo:hi], lo, d ** -0.5)
        assert torch.equal(part, full[lo:hi]), f"portion {lo}:{hi}"
        part = whole.attend(qkv[lo:hi], lo, d ** -0.5, force_split=True)
        assert torch.equal(part, full[lo:hi]), f"portion {lo}:{hi} split"
        if K().wide_supported(d, dtype, ps):
            for variant in (4, 5):
                for split in (False, True):
                    part = whole.attend(qkv[lo:hi], lo, d ** -0.5, variant=variant, force_split=split)
                    assert torch.equal(part, full[lo:hi]), f"portion {lo}:{hi}, wide kernel {variant}, split={split}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 7, 128, 300])
def test_attention_window(dtype, window):
    nq, nkv, d, ps, kv_len = 4, 2, 32, 16, 520
    qkv = rand_qkv(kv_len, nq, nkv, d, dtype, seed=window, sharp=(kv_len - window,))
    case = PagedCase(dtype, nq, nkv, d, ps, kv_len)
    dev = qkv.cuda()
    case.write(dev, 0)
    out = case.attend(dev, 0, d ** -0.5, window=window)
    q, k, v = split_qkv(qkv.double(), nq, nkv, d)
    want = naive_attention(q, k, v, 0, d ** -0.5, window=window)
    assert rel_err(out, want) < ATT_TOL[dtype]
    assert torch.equal(case.attend(dev, 0, d ** -0.5, window=window, variant=1), out)
    assert torch.equal(case.attend(dev, 0, d ** -0.5, window=window, variant=4), out)
    assert torch.equal(case.attend(dev, 0, d ** -0.5, window=window, variant=5), out)
    # pages behind the window may be gone: mark them released and decode the last rows
    for p in (kv_len - 1, 300, 130):
        first_needed = max(0, p - window + 1) // ps
        saved = case.table.clone()
        case.table[1, :first_needed] = -1
        alone = case.attend(dev[p:p + 1], p, d ** -0.5, window=window)
        coop = case.attend(dev[p:p + 1], p, d ** -0.5, window=window, variant=3)
        case.table.copy_(saved)
        lo = max(0, p - 70)                     # a portion: what its first row needs must be held
        case.table[1, :max(0, lo - window + 1) // ps] = -1
        wide = case.attend(dev[lo:p + 1], lo, d ** -0.5, window=window, variant=4)
        case.table.copy_(saved)
        assert torch.equal(alone[0], out[p]), f"row {p}"
        assert torch.equal(coop[0], out[p]), f"row {p}, cooperative kernel"
        assert torch.equal(wide, out[lo:p + 1]), f"rows {lo}..{p}, wide kernel"


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_rotation_and_cache_write(dtype):
    nq, nkv, d, ps, t, start = 6, 3, 32, 8, 21, 5
    rot = 32
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(t, (nq + 2 * nkv) * d, generator=g).to(dtype)
    qw = 1 + 0.2 * torch.randn(d, generator=g)
    kw = 1 + 0.2 * torch.randn(d, generator=g)
    eps, theta = 1e-5, 1e4
    pos = torch.arange(64, dtype=torch.float64)
    inv = 1.0 / (theta ** (torch.arange(0, rot // 2, dtype=torch.float64) * 2 / rot))
    ang = pos[:, None] * inv[None, :]
    cos, sin = ang.cos().float(), ang.sin().float()
    case = PagedCase(dtype, nq, nkv, d, ps, start + t, shuffle_seed=1)
    dev = qkv.clone().cuda()
    case.write(dev, start, qw.cuda(), kw.cuda(), eps, cos.cuda(), sin.cuda(), rot)

    q, k, v = split_qkv(qkv.double(), nq, nkv, d)

    def norm_rope(x, w):
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.double()
        c = cos[start:start + t].double()[:, None, :]
        s = sin[start:start + t].double()[:, None, :]
        lo, hi = x[..., : rot // 2], x[..., rot // 2:rot]
        return torch.cat([lo * c - hi * s, hi * c + lo * s, x[..., rot:]], dim=-1)

    tol = 1e-6 if dtype is torch.float32 else 8e-3
    got_q = dev[:, : nq * d].view(t, nq, d)
    assert rel_err(got_q, norm_rope(q, qw)) < tol
    table = case.table[1].cpu()
    want_k = norm_rope(k, kw)
    for i in range(t):
        p = start + i
        page, slot = int(table[p // ps]), p % ps
        assert rel_err(case.k_pages[page, :, slot, :], want_k[i]) < tol
        assert torch.equal(case.v_pages[page, :, :, slot].cpu().double(), v[i])
    # position 0 leaves a head untouched by the rotation (cos 1, sin 0)
    case0 = PagedCase(dtype, nq, nkv, d, ps, 1)
    one = qkv[:1].clone().cuda()
    case0.write(one, 0, None, None, eps, cos.cuda(), sin.cuda(), rot)
    assert torch.equal(one.cpu(), qkv[:1])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,ps", [(16, 8, 128, 16), (4, 4, 16, 8), (8, 1, 64, 32), (6, 2, 48, 16),
                                         (32, 2, 80, 64), (2, 2, 256, 128), (3, 3, 32, 8), (64, 8, 128, 16)])
def test_decode_attention_is_the_same_in_every_kernel(dtype, nq, nkv, d, ps):
    """The last one or two tokens of a sequence through the staged, the direct
    and the cooperative kernel, split or not: same bits, and right."""
    kv_len = 700
    qkv = rand_qkv(kv_len, nq, nkv, d, dtype, seed=d + nq, sharp=(5,))
    case = PagedCase(dtype, nq, nkv, d, ps, kv_len, shuffle_seed=7)
    dev = qkv.cuda()
    case.write(dev, 0)
    q, k, v = split_qkv(qkv.double(), nq, nkv, d)
    want = naive_attention(q, k, v, 0, d ** -0.5)
    g = nq // nkv
    for start, n in ((699, 1), (698, 2), (255, 1), (256, 1), (0, 1), (127, 2)):
        if n * g > 16:
            n = 1
        ref = case.attend(dev[start:start + n], start, d ** -0.5, variant=1, force_split=False)
        assert rel_err(ref, want[start:start + n]) < ATT_TOL[dtype], (start, n)
        variants = [(0, True), (0, False), (1, True)]
        if K().coop_supported(d, dtype, ps):
            variants += [(3, True), (3, False)]
        if K().wide_supported(d, dtype, ps):
            variants += [(4, True), (4, False)]
        for variant, split in variants:
            got = case.attend(dev[start:start + n], start, d ** -0.5, variant=variant, force_split=split)
            assert torch.equal(got, ref), f"start={start} n={n} variant={variant} split={split}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,ps", [(16, 8, 128, 16), (4, 4, 16, 8), (6, 2, 48, 16), (3, 3, 32, 8),
                                         (64, 8, 128, 16)])
def test_cooperative_items_of_several_splits_leave_the_same_partial_results(dtype, nq, nkv, d, ps):
    """A long request cut into work items of one, two, three or four splits each (a partial result a
    split, folded by the combine kernel), laid out for more splits than it has, with and without
    a window: the bits of one workgroup walking the whole request."""
    if not K().coop_supported(d, dtype, ps):
        pytest.skip("the cooperative kernel's tiles do not fit")
    kv_len = 1400                                     # six splits, the last one partly filled
    qkv = rand_qkv(kv_len, nq, nkv, d, dtype, seed=3 * d + nq, sharp=(9,))
    case = PagedCase(dtype, nq, nkv, d, ps, kv_len, shuffle_seed=5)
    dev = qkv.cuda()
    case.write(dev, 0)
    for window in (0, 700):
        for start in (1399, 1279, 1024, 511):
            ref = case.attend(dev[start:start + 1], start, d ** -0.5, window=window, variant=3, force_split=False)
            for span, pad in ((1, 0), (2, 0), (3, 1), (4, 0), (4, 3), (8, 0)):
                for few in (False, True):
                    got = case.attend(dev[start:start + 1], start, d ** -0.5, window=window, variant=3,
                                      force_split=True, span=span, pad_splits=pad, few_rows=few)
                    assert torch.equal(got, ref), f"start={start} window={window} span={span} pad={pad} few={few}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,ps", [(16, 8, 128, 16), (4, 4, 16, 8), (6, 2, 48, 16), (2, 1, 256, 16),
                                         (64, 8, 128, 16)])
def test_the_fold_for_few_rows_has_the_bits_of_the_general_fold_over_many_splits(dtype, nq, nkv, d, ps):
    """Forty-one splits (more than two of the fold's rounds of sixteen), one and three tokens."""
    if not K().coop_supported(d, dtype, ps):
        pytest.skip("the cooperative kernel's tiles do not fit")
    kv_len = 256 * 40 + 77
    qkv = rand_qkv(kv_len, nq, nkv, d, dtype, seed=5 * d + nq, sharp=(300,))
    case = PagedCase(dtype, nq, nkv, d, ps, kv_len, shuffle_seed=6)
    dev = qkv.cuda()
    case.write(dev, 0)
    for tokens in (1, 3):
        if tokens * (nq // nkv) > 16:
            continue
        start = kv_len - tokens
        ref = case.attend(dev[start:], start, d ** -0.5, variant=3, force_split=False)
        for span in (1, 5):
            general = case.attend(dev[start:], start, d ** -0.5, variant=3, force_split=True, span=span)
            few = case.attend(dev[start:], start, d ** -0.5, variant=3, force_split=True, span=span, few_rows=True)
            assert torch.equal(general, ref) and torch.equal(few, ref), f"tokens={tokens} span={span}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_fold_for_few_rows_is_right_when_it_is_handed_more_rows_than_it_was_promised(dtype):
    """The caller says "at most 16 rows" and a request brings 24 and 40: the fold notices and takes the
    general way (it used to leave the rows beyond the sixteenth unwritten)."""
    nq, nkv, d, ps = 8, 1, 64, 16
    kv_len = 900
    qkv = rand_qkv(kv_len, nq, nkv, d, dtype, seed=77, sharp=(40,))
    case = PagedCase(dtype, nq, nkv, d, ps, kv_len, shuffle_seed=2)
    dev = qkv.cuda()
    case.write(dev, 0)
    for tokens in (3, 5):
        start = kv_len - tokens
        ref = case.attend(dev[start:], start, d ** -0.5, variant=0, force_split=False)
        lied = case.attend(dev[start:], start, d ** -0.5, variant=0, force_split=True, few_rows=True)
        assert not torch.isnan(lied).any() and torch.equal(lied, ref), tokens


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,ps,rot,normed,window", [
    (16, 8, 128, 16, 128, True, 0), (64, 8, 128, 16, 128, True, 0), (8, 1, 64, 32, 64, True, 0), (4, 4, 16, 8, 16, True, 0),
    # sixteen query heads a kv head: with the new key and value more heads than a workgroup has groups of sixteen lanes
    (16, 1, 64, 16, 64, True, 0), (30, 2, 32, 8, 16, True, 0),
    (6, 2, 48, 16, 32, False, 0), (4, 2, 32, 8, 0, True, 0), (4, 2, 64, 16, 64, True, 200)])
def test_fused_decode_attention_equals_the_separate_kernels(dtype, nq, nkv, d, ps, rot, normed, window):
    """A decoded token through qk_rope_kv + cooperative attention, and through the one fused launch:
    the same output bits and the same cache contents, at the edges of pages, tiles and splits."""
    if not K().decode_fused_supported(d, dtype, ps):
        pytest.skip("the fused decode kernel does not fit into LDS for this head size")
    from lockstep_amd.ops import kernels

    g = torch.Generator().manual_seed(d + nq)
    total = 530
    qkv = (torch.randn(total, (nq + 2 * nkv) * d, generator=g) * 2).to(dtype).cuda()
    qw = (1 + 0.3 * torch.randn(d, generator=g)).cuda() if normed else None
    kw = (1 + 0.3 * torch.randn(d, generator=g)).cuda() if normed else None
    cos = sin = None
    if rot:
        inv = 1.0 / (1e4 ** (torch.arange(0, rot // 2, dtype=torch.float64) * 2 / rot))
        ang = torch.arange(total, dtype=torch.float64)[:, None] * inv[None, :]
        cos, sin = ang.cos().float().cuda(), ang.sin().float().cuda()
    eps = 1e-5
    tile, split = kernels().attention_geometry(d)
    for p in (0, 1, ps - 1, ps, 127, 128, 255, 256, 257, 300, 511, 512, 529):
        base = PagedCase(dtype, nq, nkv, d, ps, p + 1, shuffle_seed=p)
        if p:
            ctx_rows = qkv[:p].clone()
            base.write(ctx_rows, 0, qw, kw, eps, cos, sin, rot)
        first_needed = max(0, p - window + 1) // ps if window else 0
        base.table[1, :first_needed] = -1
        k0, v0 = base.k_pages.clone(), base.v_pages.clone()
        # separate kernels
        row = qkv[p:p + 1].clone()
        base.write(row, p, qw, kw, eps, cos, sin, rot)
        want = base.attend(row, p, d ** -0.5, window=window, variant=3)
        k_want, v_want = base.k_pages.clone(), base.v_pages.clone()
        for use_split in (True, False):
            base.k_pages.copy_(k0); base.v_pages.copy_(v0)
            lo = max(0, p - window + 1) if window else 0
            split_lo = lo // split
            n_splits = p // split + 1 - split_lo
            if use_split:
                items = [v for s_ in range(split_lo, split_lo + n_splits) for v in (0, 0, s_, s_ + 1, 0, n_splits, split_lo, 0)]
                combine = [0, 0, 0, n_splits]
            else:
                items, combine = [0, 0, split_lo, p // split + 1, -1, 0, 0, 0], []
            part_rows = max(nkv * (nq // nkv) * n_splits, 1)
            part_acc = torch.full((part_rows, d), float("nan"), dtype=torch.float32, device="cuda")
            part_ml = torch.full((part_rows, 2), float("nan"), dtype=torch.float32, device="cuda")
            out = torch.full((1, nq * d), float("nan"), dtype=dtype, device="cuda")
            from lockstep_amd.ops import pack_attention_items, pack_combine_items

            seq_row = base.seqs(p, 1).cpu().numpy()
            # the items of one tile once as they are and once with the tile's page ids inside them
            one_tile = split == tile and all(items[i + 3] - items[i + 2] == 1 for i in range(0, len(items), 8))
            for with_pages in (False, True) if one_tile and tile // ps <= 16 else (False,):
                base.k_pages.copy_(k0); base.v_pages.copy_(v0)
                part_acc.fill_(float("nan")); part_ml.fill_(float("nan")); out.fill_(float("nan"))
                ids = None
                if with_pages:
                    row_of_table = base.table[int(seq_row.reshape(-1, 8)[0, 4])].cpu().numpy()
                    ids = np.full((len(items) // 8, 16), -1, dtype=np.int64)
                    for i in range(len(items) // 8):
                        held = row_of_table[items[8 * i + 2] * (tile // ps):][: tile // ps]
                        ids[i, : len(held)] = held
                items_t = torch.from_numpy(pack_attention_items(items, seq_row, ids)).to(torch.int32).cuda()
                raw = qkv[p:p + 1].clone()
                K().attention_decode(raw, nq, nkv, d, base.k_pages, base.v_pages, ps, base.table, base.seqs(p, 1),
                                     items_t, len(items) // 8, out, part_acc, part_ml, d ** -0.5, window, qw, kw, eps,
                                     cos, sin, rot, p, True, single_tile=one_tile)
                if combine:
                    comb = torch.from_numpy(pack_combine_items(combine, seq_row)).to(torch.int32).cuda()
                    K().attention_combine(d, base.seqs(p, 1), comb, 1, nq, nkv, part_acc, part_ml, out)
                what = f"position {p}, split={use_split}, page ids in the items: {with_pages}"
                assert torch.equal(out.view(1, nq, d), want), what
                same_k = (base.k_pages == k_want) | ((base.k_pages != base.k_pages) & (k_want != k_want))
                same_v = (base.v_pages == v_want) | ((base.v_pages != base.v_pages) & (v_want != v_want))
                assert bool(same_k.all()) and bool(same_v.all()), f"cache after {what}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [1, 9, 16, 40, 200])
@pytest.mark.parametrize("inter,k", [(136, 96), (3072, 1024), (48, 260)])
def test_gemm_with_swiglu_epilogue(dtype, m, inter, k):
    """Gate and up interleaved in tiles of 16 rows, activation in the epilogue:
    equals silu(x Wg^T) * (x Wu^T); a row has the same bits at any batch size."""
    from lockstep_amd.ops import SWIGLU, interleave_gate_up

    g = torch.Generator().manual_seed(inter + k)
    x = torch.randn(m, k, generator=g).to(dtype)
    gate = (torch.randn(inter, k, generator=g) * 0.2).to(dtype)
    up = (torch.randn(inter, k, generator=g) * 0.2).to(dtype)
    w = interleave_gate_up(gate, up).cuda()
    assert w.shape[0] % 32 == 0 and torch.equal(w[16:32, :].cpu(), up[:16])
    out = torch.empty(m, inter, dtype=dtype, device="cuda")
    K().gemm(x.cuda(), w, out, SWIGLU)
    want = torch.nn.functional.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    assert rel_err(out, want) < TOL[dtype]
    one = torch.empty(1, inter, dtype=dtype, device="cuda")
    K().gemm(x[m - 1:].cuda(), w, one, SWIGLU)
    assert torch.equal(one[0], out[m - 1])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 64, 1024), (8, 272, 96), (16, 100, 3072), (5, 48, 200)])
def test_gemm_with_fused_norm_equals_norm_then_gemm(dtype, m, n, k):
    """The RMSNorm prologue of the skinny kernel gives the bits of the
    stand-alone norm kernel followed by the plain product, also with the
    SwiGLU epilogue."""
    from lockstep_amd.ops import STORE, SWIGLU, interleave_gate_up

    g = torch.Generator().manual_seed(m + n + k)
    h = (torch.randn(m, k, generator=g) * 3).cuda()
    nw = (1 + 0.2 * torch.randn(k, generator=g)).cuda()
    w = (torch.randn(n, k, generator=g) * 0.1).to(dtype).cuda()
    eps = 1e-5
    normed = torch.empty(m, k, dtype=dtype, device="cuda")
    K().rmsnorm(h, nw, normed, eps)
    want = torch.empty(m, n, dtype=dtype, device="cuda")
    K().gemm(normed, w, want, STORE)
    got = torch.empty(m, n, dtype=dtype, device="cuda")
    K().gemm(h, w, got, STORE, norm_weight=nw, eps=eps)
    assert torch.equal(got, want)
    inter = n // 2
    wi = interleave_gate_up(w[:inter].cpu(), w[inter:2 * inter].cpu()).cuda()
    want2 = torch.empty(m, inter, dtype=dtype, device="cuda")
    K().gemm(normed, wi, want2, SWIGLU)
    got2 = torch.empty(m, inter, dtype=dtype, device="cuda")
    K().gemm(h, wi, got2, SWIGLU, norm_weight=nw, eps=eps)
    assert torch.equal(got2, want2)
    from lockstep_amd.ops import KernelError
    with pytest.raises(KernelError):
        K().gemm(torch.zeros(17, k, device="cuda"), w, torch.empty(17, n, dtype=dtype, device="cuda"), STORE,
                 norm_weight=nw, eps=eps)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [1, 8, 16, 17, 40, 64, 65, 100, 200, 256])
@pytest.mark.parametrize("n,k", [(1024, 3072), (96, 520), (1024, 2048), (40, 64), (4096, 1024), (5120, 96),
                                 (1028, 4096), (16384, 64), (16388, 64),
                                 # enough column blocks and slices that workgroups walk several blocks
                                 (4104, 4096), (4104, 12288), (4200, 8192), (8200, 2048),
                                 # K of 25,600: fifteen slices of 1,792 (the last one shorter)
                                 (5120, 25600), (1032, 25600)])
def test_slice_sums_and_fused_add_norm_equal_the_separate_kernels(dtype, m, n, k):
    """gemm_slices + add_rmsnorm give the bits of gemm(ADD_F32) + rmsnorm: the residual row and the
    normalised row; also for a list of rows and for the plain addition.  More than 64 rows (several
    groups of rows walking the same weights) where the slice length has such a kernel; elsewhere the
    product says so."""
    from lockstep_amd.ops import ADD_F32

    most = K().gemm_slices_max_rows(k, dtype)
    assert most in (64, 256) and (most == 256) == (k <= (8192 if dtype is torch.bfloat16 else 4096))
    if m > most:
        with pytest.raises(RuntimeError, match="gemm_slices"):
            K().gemm_slices(torch.zeros(m, k, dtype=dtype, device="cuda"), torch.zeros(n, k, dtype=dtype, device="cuda"),
                            torch.zeros(K().gemm_slices_count(k), m, n, device="cuda"))
        return
    g = torch.Generator().manual_seed(n + k + m)
    x = torch.randn(m, k, generator=g).to(dtype).cuda()
    w = (torch.randn(n, k, generator=g) * 0.1).to(dtype).cuda()
    h0 = torch.randn(m, n, generator=g).cuda()
    weight = (1 + 0.1 * torch.randn(n, generator=g)).cuda()
    eps = 1e-5
    h_ref = h0.clone()
    K().gemm(x, w, h_ref, ADD_F32)
    y_ref = torch.empty(m, n, dtype=dtype, device="cuda")
    K().rmsnorm(h_ref, weight, y_ref, eps)
    slices = K().gemm_slices_count(k)
    partials = torch.full((slices, m, n), float("nan"), device="cuda")
    K().gemm_slices(x, w, partials)
    assert not torch.isnan(partials).any()
    h = h0.clone()
    y = torch.empty(m, n, dtype=dtype, device="cuda")
    K().add_rmsnorm(h, partials, weight, y, eps)
    assert torch.equal(h, h_ref) and torch.equal(y, y_ref)
    want = (h0.double() + x.double() @ w.double().T)
    assert rel_err(h, want) < (1e-5 if dtype is torch.float32 else 2e-2)
    h = h0.clone()
    K().add_rmsnorm(h, partials, None, None)
    assert torch.equal(h, h_ref)
    rows = torch.tensor([m - 1, 0][: min(2, m)], dtype=torch.int32).cuda()
    h = h0.clone()
    y = torch.empty(rows.shape[0], n, dtype=dtype, device="cuda")
    K().add_rmsnorm(h, partials, weight, y, eps, rows)
    assert torch.equal(y, y_ref[rows.long()])
    assert torch.equal(h[rows.long()], h_ref[rows.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,nq,nkv,d,n,splits", [(1, 16, 8, 128, 1024, 3), (8, 16, 8, 128, 1024, 4), (16, 4, 2, 64, 520, 2),
                                                 (5, 32, 8, 128, 4096, 8), (3, 6, 3, 32, 96, 5), (2, 64, 8, 128, 5120, 2),
                                                 (7, 2, 1, 256, 300, 3)])
def test_the_product_that_folds_the_splits_itself_equals_fold_then_product(dtype, m, nq, nkv, d, n, splits):
    """The per-split sums of m decoded tokens (some splits empty, with NaN where nothing may be read; one
    token with nothing but empty splits) through the combine launch and ``gemm_slices``, and through
    ``gemm_slices_folded`` alone: the same slice sums, bit for bit."""
    from lockstep_amd.ops import pack_combine_items

    k = nq * d
    if not K().gemm_slices_folded_ok(dtype, m, n, k, d, splits):
        assert dtype is torch.float32 or n * k * 2 >= 64 << 20, "refused although the plain slice kernel would run"
        pytest.skip("the folded product does not take these sizes")
    g = torch.Generator().manual_seed(m * 100 + nq + d + splits)
    rows = m * nq * splits
    acc = torch.randn(rows, d, generator=g) * 3
    ml = torch.stack([torch.randn(rows, generator=g) * 4, torch.rand(rows, generator=g) * 50 + 0.01], dim=1)
    empty = torch.rand(rows, generator=g) < 0.25
    empty.view(m, nq, splits)[m - 1] = True                     # the last token saw no key at all
    ml[empty, 0], ml[empty, 1] = -1e30, 0.0
    acc[empty] = float("nan")
    acc, ml = acc.cuda(), ml.cuda()
    w = (torch.randn(n, k, generator=g) * 0.1).to(dtype).cuda()
    seqs = torch.tensor([[i, 1, 700 + i, 701 + i, i, 0, 0, 0] for i in range(m)], dtype=torch.int32)
    items = torch.from_numpy(pack_combine_items([(i, 0, i * nq * splits, splits) for i in range(m)], seqs.numpy())).to(torch.int32)
    attn = torch.full((m, k), float("nan"), dtype=dtype, device="cuda")
    K().attention_combine(d, seqs.cuda(), items.cuda(), m, nq, nkv, acc, ml, attn, max_rows=nq // nkv)
    assert not torch.isnan(attn).any() and (attn[m - 1] == 0).all()
    slices = K().gemm_slices_count(k)
    want = torch.full((slices, m, n), float("nan"), device="cuda")
    K().gemm_slices(attn, w, want)
    got = torch.full((slices, m, n), float("nan"), device="cuda")
    K().gemm_slices_folded(acc, ml, splits, d, w, got)
    assert not torch.isnan(got).any()
    assert torch.equal(got, want)
    # and right: against the fold in float64
    a, b = acc.cpu().double().view(m, nq, splits, d), ml.cpu().double().view(m, nq, splits, 2)
    a[b[..., 1] <= 0] = 0
    top = b[..., 0].max(dim=2, keepdim=True).values
    scale = torch.where(b[..., 1] > 0, (b[..., 0] - top).exp(), torch.zeros_like(top))
    total = (b[..., 1] * scale).sum(2)
    x = (a * scale[..., None]).sum(2) / total.clamp_min(1e-300)[..., None]
    x[total <= 0] = 0
    product = x.reshape(m, k) @ w.cpu().double().T
    assert rel_err(got.sum(0), product) < (1e-4 if dtype is torch.float32 else 2e-2)
