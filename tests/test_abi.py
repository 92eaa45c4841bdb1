"""The C-ABI library without a GPU: it loads, exports every symbol include/decdec_hip.h declares, and
its host-only entry points agree with the oracle.  No compute call is made here."""
import ctypes
import os
import re

import numpy as np
import pytest

from decdec_amd import _lib
from oracle import decdec_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "decdec_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(decdec_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 25 and "decdec_dec_anyprec" in names
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/decdec_hip.h but not exported"
    bound = set(_lib.SIGNATURES) | set(_lib.OTHER_SYMBOLS)
    assert set(names) == bound, (set(names) ^ bound)


def test_version_and_options():
    lib = _lib.load()
    assert lib.decdec_version() >= 100
    assert _lib.get_option("fusion") == 1
    _lib.set_option("fusion", 0); assert _lib.get_option("fusion") == 0
    _lib.set_option("fusion", 1)
    with pytest.raises(RuntimeError, match="unknown option"):
        _lib.set_option("no_such_option", 1)
    # every option the header names exists, with the documented default
    header = open(os.path.join(os.path.dirname(__file__), "..", "include", "decdec_hip.h")).read()
    block = header[header.index("/* Library options"):header.index("int decdec_set_option")]
    named = set(re.findall(r'"([a-z0-9_]+)"', block))
    defaults = {"fusion": 1, "host_noncoherent": 0, "anyprec_rpw": 0, "anyprec_tile": 0, "lutgemm_ktiles": 0,
                "sqllm_ktiles": 0, "attention_two_step": 0, "attention_single_below": 512, "fused_two_per_cu": -1, "fused_small": -1, "anyprec_rg": 0, "dec_block_waves": 16,
                "dec_max_chunk_groups": 0, "gemv_max_k_ranges": 0, "dec_force_cg": 0, "dec_force_sg": 0, "dec_trace": 0,
                "dec_rows_in_flight": 0}
    assert named == set(defaults), named ^ set(defaults)
    for name, value in defaults.items():
        assert _lib.get_option(name) == value, name
    # the options a caller is meant to touch are listed apart from the tuning aids
    public = block[:block.index("Experimental")]
    assert set(re.findall(r'"([a-z0-9_]+)"', public)) == {"fusion", "dec_max_chunk_groups", "gemv_max_k_ranges", "host_noncoherent"}


@pytest.mark.parametrize("dt,code", [("fp16", 1), ("bf16", 2), ("fp32", 0)])
def test_library_floors_match_oracle_bitwise(dt, code):
    lib = _lib.load()
    rng = np.random.default_rng(3)
    out = (ctypes.c_float * 32)()
    for _ in range(500):
        a = float(O._rounder(dt)(np.float32(abs(rng.standard_normal()) * 10.0 ** rng.integers(-3, 3))))
        b = float(O._rounder(dt)(np.float32(a * rng.random())))
        _lib.check(lib.decdec_bucket_floors(a, b, code, out))
        want = O.bucket_floors(a, b, dt)
        assert np.array_equal(np.array(out[:], dtype=np.float32).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("K,N,n_tb,k_chunk", [(4096, 4096, 8, 32), (4096, 14336, 16, 32), (5120, 35840, 8, 32),
                                              (17920, 5120, 16, 64), (28672, 8192, 32, 16), (4096, 1024, 64, 8)])
def test_library_reference_geometry_matches_oracle(K, N, n_tb, k_chunk):
    info = _lib.ConfigInfo()
    _lib.check(_lib.load().decdec_reference_geometry(K, N, n_tb, k_chunk, 1, 65536, ctypes.byref(info)))
    want = O.dec_geometry(K, N, n_tb, k_chunk, 2, 65536)
    for key in _lib.REFERENCE_KEYS:
        assert getattr(info, key) == want[key], key


@pytest.mark.parametrize("waves", [4, 8, 16])
def test_dec_launch_plan_covers_the_layer(waves):
    """The DEC launch plan (host-only): every chunk and every 64-word column segment belongs to a workgroup, the row
    list holds a chunk group's picks, LDS stays within the budget, the workgroup budget is kept wherever a plan
    within it exists, and at decode shapes a workgroup fetches its segments in one batch."""
    lib = _lib.load()
    info = _lib.ConfigInfo()
    for K in (1024, 1536, 4096, 5120, 8192, 11008, 14336, 17920, 28672):
        for N in (8, 64, 1032, 4096, 7680, 14336, 28672, 35840):
            for n_tb in (1, 8, 16, 32, 64):
                for k_chunk in (1, 4, 32, 100, 1024):
                    _lib.check(lib.decdec_dec_launch_plan(K, N, n_tb, k_chunk, waves, ctypes.byref(info)))
                    chunks, nseg = -(-K // 1024), -(-(N // 8) // 64)
                    cg, sg = info.hip_chunk_groups, info.hip_segment_groups
                    assert 1 <= cg <= chunks and 1 <= sg <= nseg and info.hip_dec_blocks == cg * sg
                    cpb, spb = -(-chunks // cg), -(-nseg // sg)
                    assert info.hip_slots_per_block >= cpb * k_chunk and info.hip_slots_per_block % 2 == 0
                    teams = 4 if waves == 16 else waves // 2
                    red = max(waves * 2048, teams * (36 + 4 + 2 * 128 + 4) * 4)
                    assert info.hip_lds_bytes == info.hip_slots_per_block * 8 + 4096 + red <= 60 * 1024
                    budget = n_tb * (16 // waves)
                    assert cg * sg <= budget or cg == 1 or chunks > budget, (K, N, n_tb, k_chunk, cg, sg)
                    if k_chunk <= 32 and budget >= chunks * -(-nseg // waves):
                        assert spb <= waves, (K, N, n_tb, k_chunk, cg, sg)


MAX_CHUNK_GROUPS = 4

CONFIG_SHAPES = [(4096, 4096), (4096, 1024), (4096, 14336), (14336, 4096), (4096, 6144), (4096, 28672),      # Llama-3-8B
                 (5120, 7680), (5120, 5120), (5120, 35840), (17920, 5120),                                   # Phi-3-medium
                 (8192, 8192), (8192, 1024), (8192, 28672), (28672, 8192)]                                   # Llama-3-70B


@pytest.mark.parametrize("waves", [4, 8, 16])
def test_dec_launch_plan_bounds_the_atomic_adds_per_output(waves):
    """Every chunk group of a DEC launch adds its partial sum to an output with one atomic add (one more rounding of a
    16-bit output, in run-to-run varying order); the reference adds once (dec.cu:263-276).  The plan keeps the chunk
    groups within a small bound at every configuration shape, workgroup size and workgroup budget."""
    lib = _lib.load()
    info = _lib.ConfigInfo()
    for K, N in CONFIG_SHAPES:
        for n_tb in (8, 16, 32, 64):
            for k_chunk in (1, 8, 16, 32, 64):
                _lib.check(lib.decdec_dec_launch_plan(K, N, n_tb, k_chunk, waves, ctypes.byref(info)))
                assert 1 <= info.hip_chunk_groups <= MAX_CHUNK_GROUPS, (K, N, n_tb, k_chunk, info.hip_chunk_groups)
                assert info.hip_dec_blocks <= max(n_tb * (16 // waves), info.hip_chunk_groups)
    # the option lowers the bound (1 = the reference's single add per output)
    _lib.set_option("dec_max_chunk_groups", 1)
    try:
        for K, N in CONFIG_SHAPES:
            _lib.check(lib.decdec_dec_launch_plan(K, N, 32, 32, waves, ctypes.byref(info)))
            assert info.hip_chunk_groups == 1
    finally:
        _lib.set_option("dec_max_chunk_groups", 0)
    # only a row list that cannot fit in LDS otherwise lifts the bound (select-all at a 70B input width)
    _lib.check(lib.decdec_dec_launch_plan(28672, 8192, 32, 1024, waves, ctypes.byref(info)))
    assert info.hip_chunk_groups > MAX_CHUNK_GROUPS and info.hip_lds_bytes <= 60 * 1024


LLAMA3_8B_MODULES = {"qkv": (4096, 6144), "o": (4096, 4096), "gu": (4096, 28672), "d": (14336, 4096)}


@pytest.mark.parametrize("module", sorted(LLAMA3_8B_MODULES))
def test_fused_form_and_plan_are_monotone_in_k_chunk(module):
    """What a fused any-precision launch looks like as k_chunk grows from 1 to 12 at the Llama-3-8B module shapes
    (the autotuner's sweep): the kernel instance only ever moves from the forms chosen while the GEMV is the longer
    role (both roles in the GEMV's small workgroups, then two 1024-thread workgroups per compute unit) to the one
    chosen when DEC is (one workgroup per unit), never back; and the DEC launch plan never shrinks (workgroups,
    segment groups).  A timing cliff at one k_chunk between two cheaper neighbours therefore cannot come from the
    choice of form or plan: at 14336 -> 4096, k_chunk 6, it came from the selection itself (a window of 65 .. 128
    channels, which the 8-wave form used to hand to the general path)."""
    lib = _lib.load()
    K, N = LLAMA3_8B_MODULES[module]
    form = ctypes.c_int(0)
    info = _lib.ConfigInfo()
    order = {2: 0, 1: 1, 0: 2}                       # small workgroups -> two per unit -> one per unit
    forms, plans = [], []
    for k_chunk in range(1, 13):
        _lib.check(lib.decdec_fused_launch_form(0, 3, K, N, k_chunk, ctypes.byref(form)))
        forms.append(form.value)
        waves = {2: 8, 1: 16, 0: 16}[form.value]
        _lib.check(lib.decdec_dec_launch_plan(K, N, 32, k_chunk, waves, ctypes.byref(info)))
        plans.append((form.value, info.hip_dec_blocks, info.hip_segment_groups, info.hip_chunk_groups))
    assert all(order[a] <= order[b] for a, b in zip(forms, forms[1:])), forms
    for (fa, ba, sa, ca), (fb, bb, sb, cb) in zip(plans, plans[1:]):
        if fa == fb:
            assert bb >= ba and sb >= sa and cb >= ca, plans
    if module == "d":
        assert forms[0] == 2 and forms[5] == 2          # the down projection starts in its 8-wave form, also at k_chunk 6
    # the forced settings are honoured
    for opt, val, want in (("fused_small", 0, {0, 1}), ("fused_two_per_cu", 0, {0, 2}), ("fused_two_per_cu", 1, {1, 2})):
        _lib.set_option(opt, val)
        try:
            got = set()
            for k_chunk in range(1, 13):
                _lib.check(lib.decdec_fused_launch_form(0, 3, K, N, k_chunk, ctypes.byref(form)))
                got.add(form.value)
            assert got <= want, (opt, val, got)
        finally:
            _lib.set_option(opt, -1)


def test_invalid_handles_and_arguments_fail_cleanly():
    lib = _lib.load()
    assert lib.decdec_destroy_dec_config(12345) != 0 and "invalid DECConfig handle" in _lib.last_error()
    assert lib.decdec_destroy_dec_context(12345) != 0 and "invalid DECContext handle" in _lib.last_error()
    assert lib.decdec_dec(0, None, None, 1, 8, 8, None) != 0
    h = ctypes.c_uint64(0)
    assert lib.decdec_create_dec_config(777, 8, 1, None, 0, None, 0, None, 8, 8, ctypes.byref(h)) != 0
    # plan-time validation of the GEMVs happens before any HIP call
    buf = (ctypes.c_uint32 * 64)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.decdec_anyprec_gemv(p, p, p, p, 2, 1, 1024, 8, None) != 0 and "Bitwidth must be between 3 and 8" in _lib.last_error()
    assert lib.decdec_anyprec_gemv(p, p, p, p, 3, 0, 1024, 8, None) != 0 and "does not support float" in _lib.last_error()
    assert lib.decdec_anyprec_gemv(p, p, p, p, 3, 1, 1000, 8, None) != 0 and "multiple of 32" in _lib.last_error()
    assert lib.decdec_sqllm_gemv(p, p, p, p, 5, 1, 1024, 8, None) != 0 and "Bitwidth must be 3 or 4" in _lib.last_error()
    assert lib.decdec_lutgemm_gemv(p, p, p, p, p, 9, 128, 1, 1024, 8, None) != 0 and "between 1 and 8" in _lib.last_error()
    assert lib.decdec_lutgemm_gemv(p, p, p, p, p, 3, 48, 1, 1024, 8, None) != 0 and "group_size" in _lib.last_error()


def test_kernel_register_budgets():
    """The launch logic counts on register budgets (two 1024-thread workgroups per compute unit for the budgeted
    fused instances, no scratch in the decode-path kernels); the build records what the compiler reports."""
    import json
    from decdec_amd import build
    if not os.path.exists(build.RESOURCES_PATH):
        pytest.skip("library was not built in this tree")
    kernels = json.load(open(build.RESOURCES_PATH))
    assert len(kernels) > 40 and any("dec_sqllm_kernel" in k for k in kernels)
    assert build.check_resources(kernels) == []
    # the checker does flag what it is meant to flag
    broken = {"_ZN6decdec16dec_sqllm_kernelILi1ELb1EEEvNS_9DecParamsEjNS_11SqllmParamsE":
              {"occupancy": 8, "scratch": 68, "sgprs": 78, "vgprs": 64}}
    assert len(build.check_resources(broken)) >= 1

