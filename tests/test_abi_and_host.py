"""CPU-side checks: the C ABI library loads and exports what include/moe_a2a.h
declares, argument errors are reported before anything is launched, and the
host layer (input generator, shape checks, loud failure without a GPU) behaves."""
import ctypes as C
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from amd_distributed_2025_amd import _lib
from amd_distributed_2025_amd.task import (TASK_YML_BENCHMARKS, TASK_YML_TESTS, WORKLOADS, MoEConfig,
                                           generate_input, generate_world)

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "moe_a2a.h").read_text()


def declared_functions():
    names = re.findall(r"^(?:int|const char\*)\s+(moe_a2a_\w+)\s*\(", HEADER, flags=re.M)
    assert len(names) >= 8
    return names


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), name
    bound = set(_lib.SIGNATURES) | set(_lib.STRING_FUNCTIONS)
    assert bound == set(declared_functions())
    assert lib.moe_a2a_version().decode().startswith("moe_a2a")
    # the library on disk was built from the sources on disk
    from amd_distributed_2025_amd.build import source_id
    assert lib.moe_a2a_build_id().decode() == source_id()


def test_argument_counts_match_the_header():
    """ctypes signatures and header prototypes must list the same number of parameters."""
    flat = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    for name, args in {**_lib.SIGNATURES, **_lib.STRING_FUNCTIONS}.items():
        proto = re.search(name + r"\s*\((.*?)\);", flat, flags=re.S).group(1)
        n = 0 if proto.strip() == "void" else proto.count(",") + 1
        assert n == len(args), (name, n, len(args))


def test_integration_notes_bind_the_current_argument_lists():
    """The ctypes stub printed in the integration notes must list as many arguments as the header."""
    text = (ROOT / "INTEGRATION.md").read_text()
    found = dict(re.findall(r"lib\.(moe_a2a_\w+)\.argtypes\s*=\s*\[(.*?)\]", text))
    assert found, "no argtypes lines found"
    for name, args in found.items():
        assert len([a for a in args.split(",") if a.strip()]) == len(_lib.SIGNATURES[name]), name


@pytest.mark.parametrize("compiler,std,suffix", [("gcc", "-std=c99", ".c"), ("g++", "-std=c++11", ".cpp")])
def test_header_is_plain_c_and_cxx(tmp_path, compiler, std, suffix):
    """A C or C++ caller needs nothing but the header: it must compile on its own, pedantically,
    and every declared entry point must be usable as a function pointer."""
    import shutil
    import subprocess

    if shutil.which(compiler) is None:
        pytest.skip(f"{compiler} not installed")
    src = tmp_path / ("use_header" + suffix)
    uses = "\n".join(f"  (void)&{name};" for name in declared_functions())
    src.write_text('#include "moe_a2a.h"\nint main(void) {\n  moe_a2a_shape s = {8, 0, 256, 8, 7168, 256};\n'
                   "  (void)s;\n" + uses + "\n  return MOE_A2A_OK;\n}\n")
    r = subprocess.run([compiler, std, "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only",
                        f"-I{ROOT / 'include'}", str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_shape_struct_layout_matches_header():
    fields = re.search(r"typedef struct moe_a2a_shape \{(.*?)\} moe_a2a_shape;", HEADER, flags=re.S).group(1)
    names = re.findall(r"int32_t\s+(\w+);", fields)
    assert names == [f[0] for f in _lib.Shape._fields_]
    assert C.sizeof(_lib.Shape) == 4 * len(names)


def test_bad_arguments_are_rejected_without_touching_the_gpu():
    lib = _lib.load()
    ok = _lib.Shape(8, 0, 256, 8, 7168, 256)
    assert lib.moe_a2a_strerror(0) == b"ok"
    for status in (-1, -2, -3, -99):
        assert lib.moe_a2a_strerror(status)
    one = C.c_void_p(16)  # never dereferenced: every call below fails validation first
    # null shape / bad shapes
    assert lib.moe_a2a_dispatch_send(None, one, one, 1, one, one, one, None, None) == -1
    for bad in (_lib.Shape(0, 0, 8, 2, 16, 4), _lib.Shape(8, 8, 8, 2, 16, 4), _lib.Shape(8, 0, 12, 2, 16, 4),
                _lib.Shape(8, 0, 8, 0, 16, 4), _lib.Shape(8, 0, 8, 2, 0, 4), _lib.Shape(1, 0, 1 << 17, 2, 16, 4)):
        assert lib.moe_a2a_dispatch_send(C.byref(bad), one, one, 1, one, one, one, None, None) == -1
    # token count beyond capacity, null buffers, odd alignment, bad dtype, bad ranks
    assert lib.moe_a2a_dispatch_send(C.byref(ok), one, one, 257, one, one, one, None, None) == -1
    assert lib.moe_a2a_dispatch_send(C.byref(ok), None, one, 4, one, one, one, None, None) == -1
    assert lib.moe_a2a_dispatch_send(C.byref(ok), C.c_void_p(17), one, 4, one, one, one, None, None) == -2
    assert lib.moe_a2a_dispatch_recv(C.byref(ok), one, one, None, 4, 4, one, one, one, None, None) == -1
    assert lib.moe_a2a_dispatch_recv(C.byref(ok), one, one, one, 4, -1, one, one, one, None, None) == -1
    assert lib.moe_a2a_dispatch_recv(C.byref(ok), one, one, one, 4, 1 << 30, one, one, one, None, None) == -1
    assert lib.moe_a2a_dispatch_recv(C.byref(ok), None, one, one, 0, 4, one, one, one, None, None) == -1
    where = C.c_void_p(123)
    assert lib.moe_a2a_dispatch_recv_static(C.byref(ok), one, one, one, 4, 4, one, one, one, None, None) == -1
    assert lib.moe_a2a_dispatch_recv_static(None, one, one, one, 4, 4, one, one, one, C.byref(where), None) == -1
    # beyond the static buffer: more than 64 local experts, more than 64 ranks
    for big in (_lib.Shape(8, 0, 8 * 65, 8, 64, 16), _lib.Shape(128, 0, 128, 2, 64, 16)):
        where.value = 123
        assert lib.moe_a2a_dispatch_recv_static(C.byref(big), one, one, one, 4, 4, one, one, one,
                                                C.byref(where), None) == -4
        assert where.value is None  # no plan address is handed out with an error
    assert b"static buffer" in lib.moe_a2a_strerror(-4)
    assert lib.moe_a2a_combine_send(C.byref(ok), one, one, one, -1, 4, one, one, one, None, None) == -1
    assert lib.moe_a2a_combine_send(C.byref(ok), one, one, one, 4, -1, one, one, one, None, None) == -1
    assert lib.moe_a2a_combine_send(C.byref(ok), one, one, one, 4, 4, None, one, one, None, None) == -1
    assert lib.moe_a2a_combine_recv(C.byref(ok), one, one, one, 4, 4, one, 4, one, 0, 7, None) == -1
    assert lib.moe_a2a_combine_recv(C.byref(ok), one, one, one, 4, -1, one, 4, one, 0, 1, None) == -1
    assert lib.moe_a2a_combine_recv(C.byref(ok), one, one, one, 4, 1 << 30, one, 4, one, 0, 1, None) == -1
    assert lib.moe_a2a_expert_scale(C.byref(ok), one, one, 4, 0, 5, one, None) == -1
    # grouped GEMM: bad dtype, negative hint, null weights, out_dim not a multiple of 32, in_dim not a
    # multiple of 8, dims below 1, odd alignment of the weights and of the bias
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, 4, one, None, 64, 64, 2, one, None) == -1
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, -1, one, None, 64, 64, 1, one, None) == -1
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, 4, None, None, 64, 64, 1, one, None) == -1
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, 4, one, None, 64, 48, 1, one, None) == -1
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, 4, one, None, 60, 64, 1, one, None) == -1
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, 4, one, None, 0, 64, 1, one, None) == -1
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, 4, one, None, 64, 0, 1, one, None) == -1
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, 4, C.c_void_p(24), None, 64, 64, 1, one, None) == -2
    assert lib.moe_a2a_expert_gemm(C.byref(ok), one, one, 4, one, C.c_void_p(20), 64, 64, 1, one, None) == -2
    # dense product: negative m, null weight, n not a multiple of 32, k not a multiple of 8, odd bias pointer
    assert lib.moe_a2a_linear(one, one, None, -1, 64, 64, 1, one, None) == -1
    assert lib.moe_a2a_linear(one, None, None, 4, 64, 64, 1, one, None) == -1
    assert lib.moe_a2a_linear(one, one, None, 4, 48, 64, 1, one, None) == -1
    assert lib.moe_a2a_linear(one, one, None, 4, 64, 60, 1, one, None) == -1
    assert lib.moe_a2a_linear(one, one, None, 4, 64, 64, 3, one, None) == -1
    assert lib.moe_a2a_linear(one, one, C.c_void_p(20), 4, 64, 64, 1, one, None) == -2
    assert lib.moe_a2a_linear(None, one, None, 0, 64, 64, 1, None, None) == 0
    assert lib.moe_a2a_exchange_local(8, 16, one, one, one, 8, one, one, one, 0, 4, 4, 4, None) == -1
    assert lib.moe_a2a_exchange_local(8, 16, one, one, one, 0, one, one, one, 0, 4, -1, 4, None) == -1
    assert lib.moe_a2a_exchange_local(8, 16, one, one, one, 0, one, one, one, 0, 4, 4, 1 << 30, None) == -1
    assert lib.moe_a2a_exchange_local(8, 16, one, one, one, 0, one, one, one, 0, 4, 0, 4, None) == 0  # nothing can move
    with pytest.raises(_lib.MoeA2AError, match="invalid argument"):
        _lib.call("moe_a2a_dispatch_send", None, one, one, 1, one, one, one, None, None)


def test_no_silent_cpu_fallback():
    from amd_distributed_2025_amd import HIPAllToAll, custom_kernel

    cfg = MoEConfig(8, 2, 16, 4)
    with pytest.raises(_lib.MoeA2AError):
        HIPAllToAll(cfg, 0, 1, device="cpu")
    data = generate_input(8, 2, 16, 4, seed=1, rank=0, world_size=1)
    with pytest.raises(RuntimeError, match="GPU"):
        custom_kernel(data)


def test_product_never_imports_the_oracle():
    for path in (ROOT / "amd_distributed_2025_amd").rglob("*.py"):
        text = path.read_text()
        assert "oracle" not in re.sub(r"#.*", "", text), path
    assert "oracle" not in (ROOT / "amd_distributed_2025_amd" / "csrc" / "moe_a2a.hip").read_text()


def test_generate_input_follows_the_reference_contract():
    cfg, data, rank, world = generate_input(64, 6, 2048, 32, seed=7, rank=3, world_size=8)
    assert (rank, world) == (3, 8) and cfg.in_dtype == torch.float16 == cfg.out_dtype
    T = data.num_tokens
    assert 1 <= T <= 31  # randint(1, max): upper end exclusive
    assert data.indices.shape == (T, 6) and data.indices.dtype == torch.int32
    assert data.weights.shape == (T, 6) and data.weights.dtype == torch.float32
    assert data.x.shape == (T, 2048) and data.x.dtype == torch.float16
    assert bool((data.weights >= 0).all()) and bool((data.weights < 1).all())
    idx = data.indices.numpy()
    assert idx.min() >= 0 and idx.max() < 64
    assert all(len(set(r)) == 6 for r in idx.tolist())
    # same seed, same data; another rank, other data
    again = generate_input(64, 6, 2048, 32, seed=7, rank=3, world_size=8)[1]
    assert torch.equal(again.x, data.x) and torch.equal(again.indices, data.indices)
    other = generate_input(64, 6, 2048, 32, seed=7, rank=4, world_size=8)[1]
    assert other.num_tokens != T or not torch.equal(other.indices, data.indices)


def test_workload_generators():
    w = generate_world(WORKLOADS["C4"], 1)
    assert len(w) == 8 and all(d.num_tokens == 256 and d.x.dtype == torch.bfloat16 for _, d, _, _ in w)
    assert np.allclose(w[0][1].weights.sum(1).numpy(), 1.0, atol=1e-5)  # softmax weights
    skew = generate_world(WORKLOADS["C5"], 1)
    ids = np.concatenate([d.indices.numpy().ravel() for _, d, _, _ in skew])
    hist = np.sort(np.bincount(ids, minlength=256))[::-1]
    assert hist[0] > 8 * hist[64]  # Zipf: the head expert is far hotter than the 65th
    assert all(len(set(r)) == 8 for _, d, _, _ in skew for r in d.indices.tolist())
    # all ranks of one job share the popularity ranking
    hot0 = np.bincount(skew[0][1].indices.numpy().ravel(), minlength=256).argmax()
    hot5 = np.bincount(skew[5][1].indices.numpy().ravel(), minlength=256).argmax()
    assert hot0 == hot5 == np.bincount(ids, minlength=256).argmax()
    assert len(TASK_YML_TESTS) == 9 and len(TASK_YML_BENCHMARKS) == 5


def test_torch_extension_wraps_every_entry_point():
    """The module built by load_inline loads without a GPU, reports the library's version, has
    one wrapper per entry point that launches work, and refuses tensors that are not on a GPU
    before anything reaches the library."""
    from amd_distributed_2025_amd import _ext
    from amd_distributed_2025_amd.build import EXT_FUNCTIONS

    m = _ext.load()
    assert m.a2a_version() == _lib.load().moe_a2a_version().decode()
    wrapped = {"moe_" + f for f in EXT_FUNCTIONS}
    # not wrapped: the message lookup, and the variant for callers that cannot allocate (it hands
    # back a raw device address, which has no torch::Tensor form); the long-stream variants are
    # what a2a_dispatch_recv / a2a_combine_recv call when they are handed the table argument
    assert wrapped == set(declared_functions()) - {"moe_a2a_strerror", "moe_a2a_build_id",
                                                   "moe_a2a_dispatch_recv_static",
                                                   "moe_a2a_dispatch_recv_long", "moe_a2a_combine_recv_long"}
    source = (ROOT / "amd_distributed_2025_amd" / "csrc" / "moe_a2a_torch.cpp").read_text()
    for f in EXT_FUNCTIONS:
        assert hasattr(m, f), f
        assert "moe_" + f + "(" in source, f  # every wrapper ends in the C ABI call of its name
    x = torch.zeros(4, 16, dtype=torch.bfloat16)
    idx = torch.zeros(4, 2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="x: must be a GPU tensor"):
        m.a2a_dispatch_send([1, 0, 8, 2, 16, 4], x, idx, 4, torch.zeros(8, 16, dtype=torch.bfloat16),
                            torch.zeros(8, 5, dtype=torch.int32), torch.zeros(1, dtype=torch.int32), None, 0)
    with pytest.raises(RuntimeError, match="shape: expected"):
        m.a2a_dispatch_send([1, 0, 8], x, idx, 4, x, idx, idx, None, 0)


def test_unknown_binding_is_refused():
    from amd_distributed_2025_amd import _binding

    with pytest.raises(ValueError, match="unknown binding"):
        _binding.get("cffi")
    assert _binding.get("ctypes").version().startswith("moe_a2a")
    assert _binding.get("ext").version() == _binding.get("ctypes").version()
