"""CPU-side checks of the C-ABI boundary: the library loads, exports every symbol the header
declares, and its host-only planning entry points behave (no GPU work is launched here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rlk_hip.h")


@pytest.fixture(scope="module")
def native():
    from rl_kernel_amd import _native

    if not os.path.exists(_native.LIB_PATH):
        import importlib

        importlib.import_module("rl_kernel_amd.build").build()
    return _native


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rlk_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_something():
    names = declared_symbols()
    assert "rlk_linear_logp_fwd" in names and "rlk_linear_logp_bwd" in names


def test_library_exports_every_declared_symbol(native):
    lib = ctypes.CDLL(native.LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, f"declared in include/rlk_hip.h but not exported: {missing}"


def test_binding_covers_every_declared_symbol(native):
    assert sorted(native.SIGNATURES) == declared_symbols()
    lib = native.load()
    assert lib.rlk_version() >= 100
    assert lib.rlk_last_error() is not None


def _plan(lib, n, h, v, dtype=0, budget=0):
    out = (ctypes.c_int64 * 5)()
    assert lib.rlk_linear_logp_bwd_plan(n, h, v, dtype, budget, out) == 0
    return tuple(out)


def test_backward_workspace_is_bounded_in_token_count(native):
    lib = native.load()
    sizes = []
    for n in (32768, 65536, 131072, 262144, 1 << 20):
        need = ctypes.c_size_t(0)
        assert lib.rlk_linear_logp_bwd_workspace_bytes(n, 4096, 128256, 0, 0, ctypes.byref(need)) == 0
        sizes.append(need.value)
    # scratch does not grow with G = 64 ... 2048: one dZ block (<= 256 MiB) + fp32 dH chunk
    # (<= 128 MiB) + the d_bias column sums per token tile (1 KiB per dZ tile, <= 2 MiB)
    assert max(sizes) <= (386 << 20) + 4096, sizes
    assert max(sizes) <= 1 << 30                # <= 1 GiB extra HBM
    assert sizes[0] == sizes[1] == sizes[2]     # identical for G = 64, 128, 256
    need = ctypes.c_size_t(0)
    assert lib.rlk_linear_logp_bwd_workspace_bytes(131072, 2048, 151936, 1, 0, ctypes.byref(need)) == 0
    assert need.value <= 1 << 30


@pytest.mark.parametrize("n,h,v", [(32768, 4096, 128256), (65536, 4096, 128256),
                                   (131072, 2048, 151936), (300, 64, 1000), (1 << 20, 4096, 128256)])
@pytest.mark.parametrize("budget", [0, 64 << 20, 1 << 30])
def test_backward_plan_covers_the_problem_within_budget(native, n, h, v, budget):
    lib = native.load()
    tok_chunk, v_piece, n_chunks, n_pieces, dh_parts = _plan(lib, n, h, v, 0, budget)
    assert dh_parts in (1, 2, 4, 8)
    assert tok_chunk % 256 == 0 and v_piece % 256 == 0 and tok_chunk > 0 and v_piece > 0
    assert tok_chunk * n_chunks >= n > tok_chunk * (n_chunks - 1)
    assert v_piece * n_pieces >= v > v_piece * (n_pieces - 1)
    assert tok_chunk * v_piece * 2 <= (budget or 256 << 20)
    assert _plan(lib, n, h, v, 0, budget) == (tok_chunk, v_piece, n_chunks, n_pieces, dh_parts)  # memoised


def _dh_parts(ct, pt, ht):
    """The library's rule for the side-by-side parts of a dH launch (restated from its text in
    include/rlk_hip.h and the kernel file: at most 128 tiles, a vocab range of at least 32 tiles,
    a power of two up to 8 that keeps the launch within 256 workgroups and 16 tiles per part)."""
    tiles, parts = ct * ht, 1
    if tiles <= 128 and pt >= 32:
        lim = min(256 // tiles, pt // 16, 8)
        while parts * 2 <= lim:
            parts *= 2
    return parts


def test_backward_workspace_holds_the_dh_slots_of_every_block_kind(native):
    """A shorter last chunk or piece picks its own dH part count; the workspace must hold the fp32
    slots of whichever (chunk, piece) kind needs most, next to the dZ block, the fp32 dH
    accumulator and the d_bias column sums."""
    import random

    lib = native.load()
    rng = random.Random(7)
    for _ in range(400):
        n = rng.randrange(1, 140) * 256 - rng.randrange(0, 256)
        h = rng.choice((64, 256, 896, 1024, 2048, 4096, 8192))
        v = rng.randrange(300, 160000)
        budget = rng.choice((0, 16 << 20, 64 << 20, 128 << 20))
        tok_chunk, v_piece, n_chunks, n_pieces, parts_full = _plan(lib, n, h, v, 0, budget)
        ct, pt, ht = tok_chunk // 256, v_piece // 256, (h + 255) // 256
        n_t, v_t = (n + 255) // 256, (v + 255) // 256
        ct_last, pt_last = n_t - (n_chunks - 1) * ct, v_t - (n_pieces - 1) * pt
        assert parts_full == _dh_parts(ct, pt, ht)
        slots = 0
        for c in (ct, ct_last):
            for p_ in (pt, pt_last):
                k = _dh_parts(c, p_, ht)
                if k > 1:
                    slots = max(slots, k * c * 256 * h * 4)
        need = ctypes.c_size_t(0)
        assert lib.rlk_linear_logp_bwd_workspace_bytes(n, h, v, 0, budget, ctypes.byref(need)) == 0
        dz = tok_chunk * v_piece * 2
        acc = tok_chunk * h * 4 if n_pieces > 1 else 0
        db = ct * v_piece * 4
        assert need.value >= 256 + dz + acc + slots + db, (n, h, v, budget)
        assert slots <= 67 << 20  # <= 256 tiles of fp32


def test_forward_workspace_is_small(native):
    lib = native.load()
    need = ctypes.c_size_t(0)
    assert lib.rlk_linear_logp_fwd_workspace_bytes(32768, 4096, 128256, 0, ctypes.byref(need)) == 0
    assert 0 < need.value <= 64 << 20


def test_forward_split_count_fills_whole_rounds_of_the_chip(native):
    """The forward launches (token blocks x vocab splits) workgroups, one per CU at a time.  For any
    token count the split count must not leave most of a round of the 256 CUs idle: modelled
    occupancy (work / rounds x longest run) stays above 88 % from 8 token blocks on (the former
    rule fell to 68 % at 88 and 105 blocks), and the split partials stay within the 8 MiB of the
    allocation-free entry point up to 131072 tokens.  Read back through the workspace size
    (3 floats per token and split) at the Llama head, whose 501 vocab tiles are all full."""
    lib = native.load()
    tiles = 128256 // 256
    for blocks in range(8, 513):
        n = blocks * 256
        need = ctypes.c_size_t(0)
        assert lib.rlk_linear_logp_fwd_workspace_bytes(n, 4096, 128256, 0, ctypes.byref(need)) == 0
        splits = need.value // (12 * n)
        assert 1 <= splits <= 64 and need.value == 12 * n * splits
        plan = (ctypes.c_int64 * 4)()
        assert lib.rlk_linear_logp_fwd_plan(n, 4096, 128256, 0, plan) == 0
        assert tuple(plan) == (blocks, splits, 0, 8)
        run = -(-tiles // splits)
        rounds = -(-(blocks * splits) // 256)
        assert blocks * tiles / 256 / (rounds * run) > 0.88, (blocks, splits)
        assert need.value <= 8 << 20


def test_bad_arguments_are_reported_not_launched(native):
    lib = native.load()
    need = ctypes.c_size_t(0)
    assert lib.rlk_linear_logp_fwd_workspace_bytes(0, 4096, 128256, 0, ctypes.byref(need)) == -1
    assert b"workspace" in lib.rlk_last_error()
    # null pointers / unsupported dtype are rejected on the host before any launch
    rc = lib.rlk_linear_logp_fwd(None, None, None, None, None, None, None, 0, 16, 64, 32, 0, 7, 1.0,
                                 0, 0, 1, None, None)
    assert rc == -2
    rc = lib.rlk_linear_logp_fwd(None, None, None, None, None, None, None, 0, 16, 60, 32, 0, 0, 1.0,
                                 0, 0, 1, None, None)
    assert rc == -1 and b"null pointer" in lib.rlk_last_error()
    assert lib.rlk_logp_from_logits(None, 0, None, None, 2, None, None, 4, 4, 8, None) == -1
    assert lib.rlk_grpo_loss_from_logp(None, None, None, None, 1, None, 4, 4, 0.2, 0.0, None, None,
                                       None, None, None, None, None, 0, None) == -1
    assert lib.rlk_group_advantages(None, None, 2, 1e-6, None, None) == -1
    assert lib.rlk_device_info(0, None, None) == -1 and b"rlk_device_info" in lib.rlk_last_error()
    assert lib.rlk_linear_logp_fwd_plan(16, 64, 32, 0, None) == -1
    rc = lib.rlk_linear_logp_fwd(None, None, None, None, None, None, None, 0, 16, 64, 32, 0, 0, 0.0,
                                 0, 0, 1, None, None)
    assert rc == -1 and b"temperature" in lib.rlk_last_error()


def test_missing_library_fails_loudly(native, monkeypatch, tmp_path):
    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(native.NativeLibraryError, match="no CPU or PyTorch fallback"):
        native.load()
    assert native.available() is False


def test_backward_plan_splits_dh_only_for_few_tokens(native):
    lib = native.load()
    assert _plan(lib, 32768, 4096, 128256)[4] == 1
    assert _plan(lib, 4096, 4096, 128256)[4] == 1
    assert _plan(lib, 1024, 4096, 128256)[4] == 4      # 64 dH tiles on 256 CUs
    assert _plan(lib, 2048, 4096, 128256)[4] == 2
    assert _plan(lib, 300, 64, 40000)[4] > 1


def test_header_is_plain_c(tmp_path):
    """include/rlk_hip.h must compile as C (no C++ or torch types in the boundary)."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("gcc not available")
    src = tmp_path / "use_header.c"
    src.write_text('#include "rlk_hip.h"\nint main(void) { return rlk_version() < 0; }\n')
    res = subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-fsyntax-only",
                          "-I", os.path.join(ROOT, "include"), str(src)],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


@pytest.mark.parametrize("n,h,v", [(32768, 4096, 128256), (300, 4096, 2_000_000),
                                   (2_000_000, 4096, 256), (1 << 20, 8192, 1 << 20)])
@pytest.mark.parametrize("budget", [4 << 30, 64 << 30])
def test_backward_plan_keeps_in_tile_offsets_within_32_bits(native, n, h, v, budget):
    """Budgets of 4 GiB and more are clamped to 2 GiB: the tile loaders address the rows of one
    256-row tile with 32-bit byte offsets, so 256 x (leading dimension of the dZ block) x 2 bytes
    has to stay below 2^32 whatever the caller asks for, also for few tokens x a huge vocabulary
    and for many tokens x a tiny one."""
    lib = native.load()
    tok_chunk, v_piece, n_chunks, n_pieces, _ = _plan(lib, n, h, v, 0, budget)
    assert tok_chunk * v_piece * 2 <= 2 << 30
    assert 256 * v_piece * 2 < 2 ** 32
    assert tok_chunk * n_chunks >= n and v_piece * n_pieces >= v
    need = ctypes.c_size_t(0)
    assert lib.rlk_linear_logp_bwd_workspace_bytes(n, h, v, 0, budget, ctypes.byref(need)) == 0
    # block + fp32 dH chunk <= 1.5 x 2 GiB, + the d_bias column sums (1 KiB per 128 KiB dZ tile)
    assert need.value <= (3 << 30) + (33 << 20)


def test_compiled_pytorch_binding_exports_the_reference_symbol_names(native):
    """The pybind11 extension built from csrc/rlk_torch_binding.cpp carries the names the
    reference registers in csrc/ops.cpp:75-99 (all but the attention op, which is off this path),
    and rl_kernel_amd._C binds them in place of its ctypes route."""
    from rl_kernel_amd import _C

    assert os.path.exists(os.path.join(os.path.dirname(native.LIB_PATH), "_rlk_C.so"))
    assert _C.COMPILED
    names = ["fused_logp", "fused_logp_sm90", "fused_linear_logp_sm90", "fused_logp_forward_out",
             "fused_logp_forward_fp32", "fused_logp_forward_indexed_out",
             "fused_logp_forward_indexed_fp32", "fused_logp_forward_online_out",
             "fused_logp_forward_online_fp32", "fused_logp_forward_online_indexed_out",
             "fused_logp_forward_online_indexed_fp32"]
    for name in names:
        assert hasattr(_C.compiled_module, name), name
    for name in names:
        if name != "fused_logp_sm90":
            assert getattr(_C, name) is getattr(_C.compiled_module, name), name
    assert _C.compiled_module.rlk_version() == native.load().rlk_version()
