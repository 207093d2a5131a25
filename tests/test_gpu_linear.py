"""`moe_a2a_linear`: the product a rank forms in the reference's gemm-rs task before the
reduce-scatter, `matmul(input, weight.T) + bias` (gemm-rs/reference.py:54-57).

Shapes are the per-rank ones of gemm-rs/task.yml (k there is the job's; a rank holds k/8).
Exact cases pin indexing, the bias and the K tail; random operands are held to the bound
that float32 accumulation in any order and the two roundings allow around the float64
value, which is far inside the task's own rtol = atol = 1e-2 (gemm-rs/reference.py:66)."""
import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import gemm_rs
from oracle import moe_a2a_oracle as orc
from tests.helpers import bits, from_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

TASK_TESTS, TASK_BENCHMARKS = gemm_rs.TASK_TESTS, gemm_rs.TASK_BENCHMARKS  # gemm-rs/task.yml:66-76, :80-85


def check_against_bound(out, inp, weight, bias, name, rows):
    ib, wb = bits(inp[rows]), bits(weight)
    bb = None if bias is None else bits(bias)
    exact, tol = orc.linear_bound(ib, wb, bb, name)
    got = orc.b16_to_f32(bits(out[rows]), name).astype(np.float64)
    err = np.abs(got - exact)
    worst = np.unravel_index(np.argmax(err - tol), err.shape)
    assert (err <= tol).all(), f"at {worst}: off by {err[worst]:.3e}, allowed {tol[worst]:.3e}"
    want = orc.linear(ib, wb, bb, name)
    assert (np.abs(orc.b16_to_f32(want, name).astype(np.float64) - exact) <= tol).all()
    same = float((want == bits(out[rows])).mean())
    return same


@pytest.mark.parametrize("m,n,k,has_bias,seed", TASK_TESTS + TASK_BENCHMARKS)
def test_task_shapes(m, n, k, has_bias, seed):
    print(f"linear m={m} n={n} k={k}/8 bias={has_bias}", flush=True)
    data = gemm_rs.generate_input(0, 8, m, n, k, has_bias, seed, device=DEV)
    inp, weight, bias = data
    out = torch.full((m, n), float("nan"), dtype=inp.dtype, device=DEV)
    got = gemm_rs.local_product(data, out=out)
    torch.cuda.synchronize()
    assert got.data_ptr() == out.data_ptr() and not torch.isnan(out).any()
    rng = np.random.default_rng(seed)
    rows = np.sort(rng.choice(m, size=min(m, 96), replace=False))  # a sample of rows, every column
    rows[0], rows[-1] = 0, m - 1
    same = check_against_bound(out.cpu(), inp.cpu(), weight.cpu(), None if bias is None else bias.cpu(), "bf16",
                               torch.from_numpy(rows))
    print(f"  {same:.4f} of the sampled results equal the float32 oracle to the bit", flush=True)
    assert same > 0.97
    # the task's own check against the torch expression on the device
    want = torch.matmul(inp, weight.T)
    if bias is not None:
        want = want + bias
    assert torch.allclose(out, want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
# up to 64 rows and from 8 steps of K: a workgroup's 4 or 8 waves split K among them, 32 or 64 rows at a time
@pytest.mark.parametrize("m,n,k", [(1, 32, 512), (64, 96, 520), (33, 2880, 1000), (16, 64, 1600), (64, 96, 1544),
                                   (32, 32, 3000),
                                   # else tiles of 64 x 128 (outputs that fill few compute units) ...
                                   (1, 32, 8), (64, 64, 64), (65, 64, 520), (70, 96, 72), (129, 160, 360), (300, 2880, 200), (70, 64, 1000),
                                   (200, 160, 1096),
                                   # ... of 128 x 128 (short K, or too few tiles of 256 x 256 for every unit) ...
                                   (3000, 2944, 72), (2050, 4128, 200), (4100, 2080, 8), (1000, 4128, 1096),
                                   # ... and of 256 x 256; ragged last tiles in both directions and a K tail each
                                   (3900, 4000, 1032)])
def test_small_integers_with_bias_are_exact(m, n, k, dt):
    print(f"linear integers m={m} n={n} k={k} {dt}", flush=True)
    rng = np.random.default_rng(m * n + k)
    x = rng.integers(-1, 2, (m, k))
    w = rng.integers(-1, 2, (n, k))
    b = rng.integers(-8, 9, n)
    # stray values around the operands: a K tail or a row bound that reads past its end meets NaNs
    pad = torch.full((m + 2, k), float("nan"), dtype=dt, device=DEV)
    pad[1:m + 1] = torch.from_numpy(x).to(dt)
    wpad = torch.full((n + 2, k), float("nan"), dtype=dt, device=DEV)
    wpad[1:n + 1] = torch.from_numpy(w).to(dt)
    bias = torch.from_numpy(b).to(dt).to(DEV)
    out = torch.full((m + 2, n), 777.0, dtype=dt, device=DEV)
    gemm_rs.local_product((pad[1:m + 1], wpad[1:n + 1], bias), out=out[1:m + 1])
    torch.cuda.synchronize()
    prod = (x.astype(np.float64) @ w.T.astype(np.float64)).astype(np.int64)  # exact: small integers
    want = prod + b[None, :]
    assert np.abs(want).max() <= 256 and np.abs(prod).max() <= 256  # integers both 16-bit types hold
    assert np.array_equal(out[1:m + 1].float().cpu().numpy(), want.astype(np.float32))
    assert (out[0] == 777.0).all() and (out[m + 1] == 777.0).all()
    no_bias = gemm_rs.local_product((pad[1:m + 1], wpad[1:n + 1], None))
    assert np.array_equal(no_bias.float().cpu().numpy(), prod.astype(np.float32))


def test_bias_is_added_to_the_rounded_product():
    # 1 + 2^-8 is not a bf16 value: the product 257 * 2^-8 rounds to 1.0 (ties to even) before the
    # bias 2^-7 is added, so the result is 1 + 2^-7; adding first would give 1 + 2^-8 + 2^-7 -> 1.015625
    dt = torch.bfloat16
    x = torch.zeros(1, 8, dtype=dt, device=DEV)
    w = torch.zeros(32, 8, dtype=dt, device=DEV)
    x[0, 0], x[0, 1] = 1.0, 2.0 ** -8
    w[:, 0], w[:, 1] = 1.0, 1.0
    bias = torch.full((32,), 2.0 ** -7, dtype=dt, device=DEV)
    out = gemm_rs.local_product((x, w, bias))
    want = torch.matmul(x, w.T) + bias
    assert torch.equal(out, want) and float(out[0, 0]) == 1.0 + 2.0 ** -7
    name = "bf16"
    assert np.array_equal(orc.linear(bits(x.cpu()), bits(w.cpu()), bits(bias.cpu()), name), bits(out.cpu()))


def test_both_bindings_give_the_same_bits():
    data = gemm_rs.generate_input(0, 8, 512, 4096, 12288, True, 663, device=DEV)
    a = gemm_rs.local_product(data, binding="ctypes")
    b = gemm_rs.local_product(data, binding="ext")
    assert torch.equal(a, b)


def test_arguments_are_checked():
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        gemm_rs.local_product((x, w[:, :32], None))
    with pytest.raises(ValueError):
        gemm_rs.local_product((x, w.float(), None))
    with pytest.raises(Exception, match="invalid|argument"):
        gemm_rs.local_product((x, torch.zeros(40, 64, dtype=torch.bfloat16, device=DEV), None))  # n % 32
    with pytest.raises(ValueError):
        gemm_rs.local_product((x.cpu(), w.cpu(), None))
    assert gemm_rs.custom_kernel((x, w, None)).shape == (4, 32)


@pytest.mark.parametrize("m,n,k,has_bias,seed", [(64, 2880, 2880, True, 2035), (512, 4608, 36864, False, 1597),
                                                 (2048, 4096, 7168, False, 716), (4096, 2880, 2880, True, 136)])
def test_ranks_of_a_job_sum_to_the_whole_product(m, n, k, has_bias, seed):
    """The task as a whole on one GPU: the 8 ranks' local products over their slices of K, summed by the
    stand-in reduce-scatter, against the float64 product over all of K plus 8 times the bias (every rank
    adds it before the sum, gemm-rs/reference.py:55-59), at the task's tolerance (reference.py:66) and at
    the bound the roundings to bf16 allow."""
    W = 8
    world = [gemm_rs.generate_input(r, W, m, n, k, has_bias, seed, device=DEV) for r in range(W)]
    outs = gemm_rs.run_job(world)
    whole = torch.zeros(m, n, dtype=torch.float64, device=DEV)
    size = torch.zeros(m, n, dtype=torch.float64, device=DEV)   # sum of the magnitudes that get rounded
    for inp, weight, bias in world:
        part = inp.double() @ weight.double().T
        if bias is not None:
            size += part.abs()
            part = part + bias.double()
        whole += part
        size += part.abs()
    size += whole.abs()
    for r, out in enumerate(outs):
        assert out.shape == (m // W, n) and out.dtype == torch.bfloat16
        rows = slice(r * (m // W), (r + 1) * (m // W))
        assert torch.allclose(out.double(), whole[rows], rtol=1e-2, atol=1e-2), f"rank {r}"
        # and far inside it: every value that is rounded to bf16 on the way (each rank's product, its sum
        # with the bias, the total) may be off by 2^-9 of its size; float32 sums add far less
        err = (out.double() - whole[rows]).abs()
        assert (err <= 2.0 ** -8 * size[rows] + 1e-9).all(), f"rank {r}: {float(err.max()):.3e}"
    # the ranks share the bias (drawn from the job's seed) and differ in their operands
    if has_bias:
        assert torch.equal(world[0][2], world[W - 1][2])
    assert not torch.equal(world[0][0], world[1][0])


def _random_shapes(seed):
    rng = np.random.default_rng(seed)
    shapes = []
    for lo_m, hi_m, hi_n, count in ((1, 65, 70, 12), (65, 1400, 70, 10), (1500, 4200, 140, 10)):
        for _ in range(count):
            k = 8 * int(rng.choice([rng.integers(1, 9), rng.integers(9, 64), rng.integers(64, 200)]))
            shapes.append((int(rng.integers(lo_m, hi_m)), 32 * int(rng.integers(hi_n // 2, hi_n)), k))
    return shapes


@pytest.mark.parametrize("m,n,k", _random_shapes(20251))
def test_random_shapes_of_small_integers_are_exact(m, n, k):
    """Shapes drawn at random across the ranges that pick each kernel and tile (few rows with K split over
    waves, tiles of 64 x 128, 128 x 128 and 256 x 256), ragged in every direction: small integers with a
    bias must come out exactly, with stray NaNs around the operands and sentinels around the result."""
    print(f"linear random shape m={m} n={n} k={k}", flush=True)
    dt = torch.bfloat16
    rng = np.random.default_rng(m * 7919 + n * 31 + k)
    x = rng.integers(-1, 2, (m, k))
    w = rng.integers(-1, 2, (n, k))
    b = rng.integers(-8, 9, n)
    pad = torch.full((m + 2, k), float("nan"), dtype=dt, device=DEV)
    pad[1:m + 1] = torch.from_numpy(x).to(dt)
    wpad = torch.full((n + 2, k), float("nan"), dtype=dt, device=DEV)
    wpad[1:n + 1] = torch.from_numpy(w).to(dt)
    bias = torch.from_numpy(b).to(dt).to(DEV)
    out = torch.full((m + 2, n), 777.0, dtype=dt, device=DEV)
    gemm_rs.local_product((pad[1:m + 1], wpad[1:n + 1], bias), out=out[1:m + 1])
    torch.cuda.synchronize()
    prod = (x.astype(np.float64) @ w.T.astype(np.float64)).astype(np.int64)
    want = prod + b[None, :]
    assert np.abs(want).max() <= 256 and np.abs(prod).max() <= 256
    assert np.array_equal(out[1:m + 1].float().cpu().numpy(), want.astype(np.float32))
    assert (out[0] == 777.0).all() and (out[m + 1] == 777.0).all()
