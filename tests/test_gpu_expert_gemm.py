"""The grouped GEMM over the expert-major layout (`moe_a2a_expert_gemm`), which a
model runs where all2all/reference.py:262 has its stand-in expert.

What is exact is tested exactly: weights that are signed permutations, and small
integers whose sums every summation order represents. Random operands are held to
the bound that float32 accumulation in any order plus one rounding allows around
the float64 product (`oracle.expert_gemm_bound`); the float32 oracle is inside the
same bound, and the two mostly agree to the bit."""
import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import LocalWorld, WORKLOADS
from amd_distributed_2025_amd.task import MoEConfig, dtype_name
from oracle import moe_a2a_oracle as orc
from tests.helpers import bits, from_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SENTINEL = 0x7B7B  # bit pattern rows past the counts must keep


def rank_object(W, nle, H, max_tokens, dt, binding="ctypes"):
    cfg = MoEConfig(W * nle, 1, H, max_tokens, dt, dt)
    return LocalWorld(cfg, W, device=DEV, binding=binding).ranks[W - 1], cfg


def run_gemm(a, ex, counts, w, hint=None):
    """Runs the kernel twice into the same buffer, the second time over a buffer of
    sentinels, and returns the bit patterns of that second result."""
    num = torch.tensor(counts, dtype=torch.int32, device=DEV)
    ey = a.expert_gemm(ex, num, w, rows_hint=hint)
    ey.view(torch.int16).fill_(SENTINEL)
    again = a.expert_gemm(ex, num, w, rows_hint=hint)
    assert again.data_ptr() == ey.data_ptr()
    torch.cuda.synchronize()
    return bits(again)


def check_padding_untouched(got, counts):
    for le, c in enumerate(counts):
        assert (got[le, c:] == SENTINEL).all(), f"expert {le}: rows past its {c} were written"


def ragged_counts(rng, nle, max_recv, special):
    counts = rng.integers(0, min(max_recv, 200) + 1, nle)
    for i, c in enumerate(special):
        counts[i % nle] = min(c, max_recv)
    return [int(c) for c in counts]


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("W,nle,H,max_tokens", [(1, 1, 64, 16), (1, 2, 32, 8), (2, 3, 96, 40), (2, 3, 192, 80), (4, 8, 2048, 128), (8, 2, 7168, 40)])
def test_signed_permutation_weights_move_columns_exactly(W, nle, H, max_tokens, dt):
    print(f"permutation W={W} nle={nle} H={H} T={max_tokens} {dt}", flush=True)
    rng = np.random.default_rng(H + nle)
    a, cfg = rank_object(W, nle, H, max_tokens, dt)
    max_recv = W * max_tokens
    counts = ragged_counts(rng, nle, max_recv, [0, max_recv, 1, 129, 128, 127])
    xb = rng.integers(0, 1 << 16, (nle, max_recv, H), dtype=np.uint16)
    name = dtype_name(dt)
    finite = np.isfinite(orc.b16_to_f32(xb, name))
    xb[~finite] = 0x3C00
    perm = np.stack([rng.permutation(H) for _ in range(nle)])
    sign = rng.choice([-1.0, 1.0], (nle, H))
    w = torch.zeros(nle, H, H, dtype=dt)
    for le in range(nle):
        w[le, torch.arange(H), torch.from_numpy(perm[le])] = torch.from_numpy(sign[le]).to(dt)
    got = run_gemm(a, from_bits(xb, dt).to(DEV), counts, w.to(DEV))
    check_padding_untouched(got, counts)
    for le, c in enumerate(counts):
        moved = xb[le, :c][:, perm[le]]
        want = np.where(sign[le] < 0, moved ^ 0x8000, moved).astype(np.uint16)
        # -0 + 0 sums: a zero's sign is the one thing the order of the sum may change
        zero = (want & 0x7FFF) == 0
        assert np.array_equal(got[le, :c][~zero], want[~zero]), f"expert {le}"
        assert ((got[le, :c][zero] & 0x7FFF) == 0).all()


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("H", [96, 128, 192])
def test_small_integers_sum_exactly(H, dt):
    print(f"integers H={H} {dt}", flush=True)
    rng = np.random.default_rng(H)
    W, nle, max_tokens = 2, 5, 150
    a, cfg = rank_object(W, nle, H, max_tokens, dt)
    max_recv = W * max_tokens
    counts = ragged_counts(rng, nle, max_recv, [max_recv, 0, 65])
    x = rng.integers(-1, 2, (nle, max_recv, H))
    w = rng.integers(-1, 2, (nle, H, H))
    got = run_gemm(a, torch.from_numpy(x).to(dt).to(DEV), counts, torch.from_numpy(w).to(dt).to(DEV))
    check_padding_untouched(got, counts)
    name = dtype_name(dt)
    for le, c in enumerate(counts):
        want = x[le, :c] @ w[le].T  # |sums| <= H <= 192: integers both 16-bit types hold
        assert np.array_equal(orc.b16_to_f32(got[le, :c], name), want.astype(np.float32)), f"expert {le}"
        assert np.array_equal(orc.b16_to_f32(orc.expert_gemm(bits(torch.from_numpy(x[le, :c]).to(dt)),
                                                             bits(torch.from_numpy(w[le]).to(dt)), name), name),
                              want.astype(np.float32))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("in_dim,out_dim", [(96, 160), (200, 64), (128, 128)])
def test_bias_and_unequal_widths_on_every_kernel(in_dim, out_dim, dt):
    """[nle, out_dim, in_dim] weights with a bias, small integers (every order of the sum agrees, and
    both roundings are exact): the streaming kernel (row count 0) and the tiles of 64 x 128 / 128 x 128
    and 256 x 256 (row counts of 56 and 768 per expert) all give the integers of `x @ w.T + b`."""
    print(f"bias in={in_dim} out={out_dim} {dt}", flush=True)
    rng = np.random.default_rng(in_dim * 7 + out_dim)
    W, nle, max_tokens = 1, 5, 300
    a, cfg = rank_object(W, nle, in_dim, max_tokens, dt)
    counts = ragged_counts(rng, nle, max_tokens, [max_tokens, 0, 65, 129])
    x = rng.integers(-1, 2, (nle, max_tokens, in_dim))
    w = rng.integers(-1, 2, (nle, out_dim, in_dim))
    b = rng.integers(-20, 21, (nle, out_dim))
    ex, wt, bt = (torch.from_numpy(v).to(dt).to(DEV) for v in (x, w, b))
    num = torch.tensor(counts, dtype=torch.int32, device=DEV)
    name = dtype_name(dt)
    for hint in (0, 56 * nle, 768 * nle):
        out = torch.empty(nle, max_tokens, out_dim, dtype=dt, device=DEV)
        out.view(torch.int16).fill_(SENTINEL)
        got = a.expert_gemm(ex, num, wt, bias=bt, rows_hint=hint, out=out)
        assert got.data_ptr() == out.data_ptr()
        torch.cuda.synchronize()
        got = bits(got)
        check_padding_untouched(got, counts)
        for le, c in enumerate(counts):
            want = x[le, :c] @ w[le].T + b[le][None, :]   # |values| <= 200 + 20: integers both types hold
            assert np.array_equal(orc.b16_to_f32(got[le, :c], name), want.astype(np.float32)), f"hint {hint} expert {le}"
    # the oracle's statement of the same layer
    rows = np.concatenate([x[le, :c] for le, c in enumerate(counts)])
    want = np.concatenate([x[le, :c] @ w[le].T + b[le][None, :] for le, c in enumerate(counts)])
    stated = orc.grouped_linear(bits(torch.from_numpy(rows).to(dt)), np.array(counts), bits(wt.cpu()), bits(bt.cpu()), name)
    assert np.array_equal(orc.b16_to_f32(stated, name), want.astype(np.float32))


def random_case(a, cfg, W, counts, seed, hint=None, check_experts=None):
    nle, H, dt = cfg.num_experts // W, cfg.hidden_dim, cfg.in_dtype
    max_recv = W * cfg.max_num_tokens
    g = torch.Generator(device=DEV).manual_seed(seed)
    ex = torch.randn(nle, max_recv, H, generator=g, device=DEV, dtype=torch.float32).to(dt)
    w = (torch.randn(nle, H, H, generator=g, device=DEV, dtype=torch.float32) / H ** 0.5).to(dt)
    got = run_gemm(a, ex, counts, w, hint)
    check_padding_untouched(got, counts)
    name = dtype_name(dt)
    same = total = 0
    for le in (range(nle) if check_experts is None else check_experts):
        c = counts[le]
        if c == 0:
            continue
        xb, wb = bits(ex[le, :c]), bits(w[le])
        exact, tol = orc.expert_gemm_bound(xb, wb, name)
        err = np.abs(orc.b16_to_f32(got[le, :c], name).astype(np.float64) - exact)
        worst = np.unravel_index(np.argmax(err - tol), err.shape)
        assert (err <= tol).all(), f"expert {le} at {worst}: off by {err[worst]:.3e}, allowed {tol[worst]:.3e}"
        want32 = orc.expert_gemm(xb, wb, name)
        assert (np.abs(orc.b16_to_f32(want32, name).astype(np.float64) - exact) <= tol).all()
        same += int((want32 == got[le, :c]).sum())
        total += want32.size
    print(f"  {same}/{total} results equal the float32 oracle to the bit", flush=True)
    assert same >= 0.98 * total  # they differ where the sum lies next to a rounding boundary
    return got


@pytest.mark.parametrize("name", ["C3", "C4"])
def test_random_operands_at_workload_sizes(name):
    print(f"gemm at {name}", flush=True)
    wl = WORKLOADS[name]
    W, H, T, K = wl["world_size"], wl["hidden_dim"], wl["max_num_tokens"], wl["experts_per_token"]
    nle = wl["num_experts"] // W
    dt = torch.bfloat16
    a, cfg = rank_object(W, nle, H, T, dt)
    rng = np.random.default_rng(7)
    max_recv = W * T
    # the counts a rank sees at this shape: about W*T*K/num_experts rows per expert, ragged, one empty, one hot
    counts = [int(c) for c in rng.poisson(W * T * K // wl["num_experts"], nle)]
    counts[1] = 0
    counts[2] = min(max_recv, 300)
    random_case(a, cfg, W, counts, seed=11, hint=sum(counts))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_hints_and_hot_experts(dt):
    print(f"gemm hints {dt}", flush=True)
    W, nle, H, T = 4, 6, 512, 96
    a, cfg = rank_object(W, nle, H, T, dt)
    max_recv = W * T
    counts = [max_recv, 0, 5, max_recv, 131, 64]
    full = random_case(a, cfg, W, counts, seed=3, hint=sum(counts))
    for hint in (0, 1, 200, None):  # a hint only sizes the launch: the result does not depend on it
        assert np.array_equal(run_gemm_same(a, cfg, W, counts, 3, hint), full), f"hint {hint}"


def run_gemm_same(a, cfg, W, counts, seed, hint):
    nle, H, dt = cfg.num_experts // W, cfg.hidden_dim, cfg.in_dtype
    g = torch.Generator(device=DEV).manual_seed(seed)
    ex = torch.randn(nle, W * cfg.max_num_tokens, H, generator=g, device=DEV, dtype=torch.float32).to(dt)
    w = (torch.randn(nle, H, H, generator=g, device=DEV, dtype=torch.float32) / H ** 0.5).to(dt)
    return run_gemm(a, ex, counts, w, hint)


def test_counts_above_the_padding_are_clamped():
    W, nle, H, T = 2, 2, 128, 8
    a, cfg = rank_object(W, nle, H, T, torch.bfloat16)
    got = run_gemm_same(a, cfg, W, [W * T + 50, 3], 5, None)
    want = run_gemm_same(a, cfg, W, [W * T, 3], 5, None)
    assert np.array_equal(got, want)


def test_both_bindings_give_the_same_bits():
    W, nle, H, T = 2, 4, 256, 64
    counts = [128, 7, 0, 90]
    outs = []
    for binding in ("ctypes", "ext"):
        a, cfg = rank_object(W, nle, H, T, torch.bfloat16, binding)
        outs.append(run_gemm_same(a, cfg, W, counts, 9, None))
    assert np.array_equal(outs[0], outs[1])


def test_unsupported_shapes_raise():
    a, cfg = rank_object(1, 1, 80, 4, torch.bfloat16)  # not whole wave tiles of 32 columns
    ex = torch.zeros(1, 4, 80, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(1, 80, 80, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(Exception, match="invalid|argument"):
        a.expert_gemm(ex, torch.tensor([4], dtype=torch.int32, device=DEV), w)
    with pytest.raises(ValueError, match="weights must be"):  # in_dim of the weights is not the rows'
        a.expert_gemm(ex, torch.tensor([4], dtype=torch.int32, device=DEV), w[:, :, :64].contiguous())
    with pytest.raises(ValueError, match="bias must be"):
        a.expert_gemm(ex, torch.tensor([4], dtype=torch.int32, device=DEV), w, bias=w[0, :1, :64].contiguous())


@pytest.mark.parametrize("H,width", [(576, 5), (640, 6), (704, 7), (832, 8)])
def test_wide_workgroups_of_every_width(H, width):
    """The streaming kernel between 48 and 56 rows per expert (above, the product runs on tiles): with
    blocks of 128 tokens and many tiles a workgroup is 5 to 8 waves wide, the width picked from the row
    count so that the launch fills the compute units in whole rounds: 128 experts of about 52 rows and
    these four row lengths take the four widths (5 to 7 waves leave the token loads to the first four).
    Signed permutation weights: exact."""
    print(f"wide workgroups: H={H}, expected width {width} waves", flush=True)
    dt, nle, max_tokens = torch.bfloat16, 128, 140
    rng = np.random.default_rng(H)
    a, cfg = rank_object(1, nle, H, max_tokens, dt)
    counts = [52] * nle
    for i, c in enumerate([0, 1, 129, 128, 127, 33]):   # ragged, and the total stays 52 * nle
        counts[2 + i], counts[nle - 3 - i] = c, 104 - c if c <= 104 else 0
    counts[1], counts[nle - 2] = 140, 0
    total = 52 * nle
    for i in range(20, 20 + (sum(counts) - total) // 2):
        counts[i] -= 2
    assert sum(counts) == total and 0 <= min(counts) and max(counts) <= max_tokens
    xb = rng.integers(0, 1 << 16, (nle, max_tokens, H), dtype=np.uint16)
    xb[~np.isfinite(orc.b16_to_f32(xb, "bf16"))] = 0x3C00
    perm = np.stack([rng.permutation(H) for _ in range(nle)])
    sign = rng.choice([-1.0, 1.0], (nle, H))
    w = torch.zeros(nle, H, H, dtype=dt)
    for le in range(nle):
        w[le, torch.arange(H), torch.from_numpy(perm[le])] = torch.from_numpy(sign[le]).to(dt)
    got = run_gemm(a, from_bits(xb, dt).to(DEV), counts, w.to(DEV), hint=total)
    check_padding_untouched(got, counts)
    for le, c in enumerate(counts):
        moved = xb[le, :c][:, perm[le]]
        want = np.where(sign[le] < 0, moved ^ 0x8000, moved).astype(np.uint16)
        zero = (want & 0x7FFF) == 0
        assert np.array_equal(got[le, :c][~zero], want[~zero]), f"expert {le}"
        assert ((got[le, :c][zero] & 0x7FFF) == 0).all()


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("nle,H,max_tokens,counts", [
    # about 160 rows per expert and more: tiles of 128 x 128 (ragged last tiles in both directions, an empty
    # expert, exact multiples of the tile, one row)
    (6, 416, 400, [384, 0, 5, 400, 131, 256]),
    (5, 7168, 300, [290, 213, 0, 256, 129]),
    # about 768 rows and more: tiles of 256 x 256
    (3, 320, 1100, [1100, 770, 513]),
    (2, 1024, 1030, [1025, 1024]),
])
def test_tiles_for_experts_with_hundreds_of_rows(nle, H, max_tokens, counts, dt):
    """From about 160 rows per expert (judged from the row count the caller passes) the product runs on the
    dense kernel's tiles, found over the experts from the device-side counts. The row count only picks the
    kernel and sizes the launch: every value of it gives the same bits, those of the streaming kernel
    (hint 0) included, within the float32 bound, and rows past the counts stay untouched."""
    print(f"gemm tiles nle={nle} H={H} counts={counts} {dt}", flush=True)
    a, cfg = rank_object(1, nle, H, max_tokens, dt)
    total = sum(counts)
    full = random_case(a, cfg, 1, counts, seed=21, hint=total, check_experts=[0, nle - 1] if H > 2048 else None)
    for hint in (0, 160 * nle, 768 * nle, 10 * total):
        assert np.array_equal(run_gemm_same(a, cfg, 1, counts, 21, hint), full), f"hint {hint}"


def test_graph_replays_of_both_products_match_eager():
    """The grouped product (on tiles, and the streaming kernel through a low row count) and the gemm-rs
    product captured in a HIP graph after one warm-up call each (the first call on a GPU sets kernel
    attributes): every replay, with new operands and eager work in between, gives the eager bits."""
    from amd_distributed_2025_amd import gemm_rs
    dt, nle, H, T = torch.bfloat16, 6, 512, 300
    a, cfg = rank_object(1, nle, H, T, dt)
    counts = [300, 0, 131, 64, 257, 5]
    num = torch.tensor(counts, dtype=torch.int32, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(4)
    ex = torch.randn(nle, T, H, generator=g, device=DEV).to(dt)
    w = (torch.randn(nle, H, H, generator=g, device=DEV) / H ** 0.5).to(dt)
    lin = gemm_rs.generate_input(0, 8, 512, 4096, 12288, True, 663, device=DEV)
    lin_out = torch.empty(512, 4096, dtype=dt, device=DEV)
    outs = {}

    def step():
        outs["tiles"] = a.expert_gemm(ex, num, w, rows_hint=sum(counts))
        outs["linear"] = gemm_rs.local_product(lin, out=lin_out)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(3):
        ex.copy_(torch.randn(nle, T, H, generator=g, device=DEV).to(dt))   # new operands, eager work between replays
        lin[0].mul_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_tiles, got_lin = outs["tiles"].clone(), outs["linear"].clone()
        want_tiles = a.expert_gemm(ex, num, w, rows_hint=0).clone()   # eager, the streaming kernel: the same bits
        want_lin = gemm_rs.local_product(lin).clone()
        torch.cuda.synchronize()
        for le, c in enumerate(counts):
            assert torch.equal(got_tiles[le, :c], want_tiles[le, :c]), f"replay {i}, expert {le}"
        assert torch.equal(got_lin, want_lin), f"replay {i}: linear"


def _random_layouts(seed, count):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        nle = int(rng.integers(1, 41))
        H = 32 * int(rng.integers(1, 30))
        max_tokens = int(rng.choice([40, 130, 300, 600]))
        counts = [int(c) for c in rng.integers(0, max_tokens + 1, nle)]
        for i, c in enumerate(rng.choice([0, 1, 31, 32, 33, 64, 127, 128, 129, 256, 257, max_tokens], 3)):
            counts[int(rng.integers(0, nle))] = min(int(c), max_tokens)
        cases.append((nle, H, max_tokens, counts))
    # more experts than a workgroup has threads: every thread sums the row tiles of a run of experts
    many = [int(c) for c in rng.integers(0, 131, 600)]
    many[0], many[299], many[599] = 130, 0, 129
    cases.append((600, 64, 130, many))
    return cases


@pytest.mark.parametrize("nle,H,max_tokens,counts", _random_layouts(77, 14))
def test_random_layouts_give_the_same_bits_on_every_kernel(nle, H, max_tokens, counts):
    """Random numbers of experts, row lengths and ragged counts: the streaming kernel (row count 0), tiles of
    64 x 128 or 128 x 128 (a row count of 56 per expert or the true one) and tiles of 256 x 256 (768 per
    expert) give the same bits, inside the float32 bound, and leave the rows past the counts alone."""
    print(f"gemm random layout nle={nle} H={H} T={max_tokens} rows={sum(counts)}", flush=True)
    a, cfg = rank_object(1, nle, H, max_tokens, torch.bfloat16)
    base = random_case(a, cfg, 1, counts, seed=nle * 1000 + H, hint=0, check_experts=[0, nle - 1])
    for hint in (max(sum(counts), 56 * nle), 768 * nle):
        assert np.array_equal(run_gemm_same(a, cfg, 1, counts, nle * 1000 + H, hint), base), f"hint {hint}"
