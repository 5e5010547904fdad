"""The C-ABI library loads and exports every symbol include/parrot_hip.h declares
(no compute calls: this runs without a GPU)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "parrot_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ph_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_bound_and_exported():
    from parrotserve_amd import _lib

    declared = _declared_symbols()
    assert len(declared) >= 12
    assert sorted(_lib.SIGNATURES) == declared, "ctypes table and header disagree"
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} not exported"


def test_status_strings_and_version():
    from parrotserve_amd import _lib

    lib = _lib.load()
    assert lib.ph_abi_version() >= 2
    assert _lib.status_string(0) == "ok"
    assert "head size" in _lib.status_string(_lib.PH_ERR_HEAD_DIM)
    with pytest.raises(RuntimeError):
        _lib.check(_lib.PH_ERR_DTYPE, "x")
    with pytest.raises(ValueError):
        _lib.check(_lib.PH_ERR_ARG, "x")


def test_workspace_queries_are_host_only():
    from parrotserve_amd import _lib

    lib = _lib.load()
    # C2 shape: B 64, H 32, D 128, one group, prefix 4096, suffix <= 512
    n = lib.ph_decode_workspace_bytes(64, 32, 128, 1, 4096, 512, 32, 0)
    assert n > 0 and n % 256 == 0
    assert lib.ph_decode_workspace_bytes(0, 32, 128, 1, 4096, 512, 32, 0) == 0
    assert lib.ph_decode_workspace_bytes(64, 32, 128, 1, 4096, 512, 0, 448) < n  # balanced form: fewer partial rows
    assert lib.ph_prefill_workspace_bytes(1000, 40, 128, 1, 3000) > 0
    # 32-bit elements take the row-by-row path: partials for every token
    assert lib.ph_prefill_workspace_bytes(1000, 40, 128, 2, 3000) > lib.ph_prefill_workspace_bytes(1000, 40, 128, 1, 3000)


def test_how_the_planner_divides_a_256_unit_device():
    """``ph_decode_suffix_lanes`` is host arithmetic (without a device it plans for 256 compute units): the lane
    counts behind the measured configurations, so that a change of the cost models shows up here and not only as a
    slower benchmark.  lanes = 8 waves x (256 - prefix-only workgroups) / waves per piece."""
    from parrotserve_amd import _lib

    lanes = _lib.load().ph_decode_suffix_lanes
    f16 = _lib.PH_F16
    assert lanes(64, 32, 128, f16, 1, 4096, 512, 1) == 160    # config 2: 96 prefix-only workgroups (3 splits x 32 heads)
    assert lanes(128, 40, 128, f16, 4, 6000, 1024, 1) == 119  # config 5: 107 (2 splits x 160 units in three rounds)
    assert lanes(64, 40, 128, f16, 1, 8192, 20, 1) == 12      # the reference benchmark's shape: 240 (6 splits x 40)
    # all prefix (a long prefix under a few own tokens), no prefix, no matrix-core form: every compute unit streams
    assert lanes(64, 8, 128, f16, 1, 8192, 8, 1) == 256 * 8 // 2
    assert lanes(64, 32, 128, f16, 0, 0, 512, 1) == 256
    assert lanes(64, 32, 128, _lib.PH_F32, 1, 4096, 512, 1) == 256
    assert lanes(64, 32, 256, f16, 1, 4096, 512, 1) == 256 * 8 // 16
    # grouped KV heads: long lists are streamed for four query heads at once (a piece takes a quarter of the waves);
    # short ones, and groups the grouped stream is not built for, keep one piece per four query heads
    assert lanes(64, 32, 128, f16, 1, 4096, 512, 4) > 2 * lanes(64, 32, 128, f16, 1, 4096, 512, 1)
    assert lanes(64, 32, 128, f16, 1, 4096, 60, 4) <= 256
    assert lanes(64, 32, 128, f16, 0, 0, 512, 2) == 256


def test_argument_validation_needs_no_gpu():
    """Bad arguments are rejected before any launch."""
    from parrotserve_amd import _lib

    lib = _lib.load()
    assert lib.ph_move_tokens(None, None, None, None, 0, 4, 2, 8, 3, 16, 8, 1, 16, 8, 1, None) == _lib.PH_ERR_DTYPE
    assert lib.ph_move_tokens(None, None, None, None, 0, 4, 2, 8, 2, 16, 8, 1, 16, 8, 1, None) == _lib.PH_ERR_ARG
    assert lib.ph_move_tokens(None, None, None, None, 0, 0, 2, 8, 2, 16, 8, 1, 16, 8, 1, None) == _lib.PH_OK
    assert lib.ph_rms_norm(None, None, None, 1e-6, 4, 64, 64, 64, 7, 1, None) == _lib.PH_ERR_DTYPE
    # unsupported head size mirrors the reference's "Unsupported head size" check
    rc = lib.ph_decode_attention(1, 1, 1, 1, 4, 2, 72, 0, 144, 144, 144, 1.0, 0, None, None, None, None, 0,
                                 None, None, 0, 0, None, 0, 0, None, None, 0, None)
    assert rc == _lib.PH_ERR_HEAD_DIM
    # fused per-layer ops and the table patch
    assert lib.ph_add_rms_norm(None, None, None, None, 1e-6, 4, 64, 64, 64, 64, 9, 1, None) == _lib.PH_ERR_DTYPE
    assert lib.ph_add_rms_norm(None, None, None, None, 1e-6, 4, 64, 32, 64, 64, 0, 1, None) == _lib.PH_ERR_ARG  # stride < n
    assert lib.ph_add_rms_norm(None, None, None, None, 1e-6, 0, 64, 64, 64, 64, 0, 1, None) == _lib.PH_OK       # no rows
    assert lib.ph_add_rms_norm(None, None, None, None, 1e-6, 4, 64, 64, 64, 64, 0, 1, None) == _lib.PH_ERR_ARG  # null pointers
    assert lib.ph_silu_mul(None, None, None, 4, 0, 8, 8, 8, 0, None) == _lib.PH_ERR_ARG
    assert lib.ph_silu_mul(None, None, None, 4, 8, 8, 8, 8, 5, None) == _lib.PH_ERR_DTYPE
    assert lib.ph_rope_append(None, None, None, None, None, None, None, None, 0, 4, 2, 2, 128, 130, 256, 256, 256, 256,
                              0, 1, None) == _lib.PH_ERR_ARG  # rotary size beyond the head size
    assert lib.ph_rope_append(None, None, None, None, None, None, None, None, 7, 4, 2, 2, 128, 128, 256, 256, 256, 256,
                              0, 1, None) == _lib.PH_ERR_ARG  # unknown index type
    assert lib.ph_rope_append(None, None, None, None, None, None, None, None, 0, 0, 2, 2, 128, 128, 256, 256, 256, 256,
                              0, 0, None) == _lib.PH_OK       # no tokens
    # gathers out of the block-structured layouts
    gk = lambda n, D, x, eb, idx=0: lib.ph_gather_blocked_k(None, None, None, None, idx, n, 2, D, 16, x, eb, 4096, 2048,
                                                            128, 8, 1, 256, 128, 1, None)
    assert gk(4, 128, 8, 2) == _lib.PH_ERR_ARG       # null pointers
    assert gk(0, 128, 8, 2) == _lib.PH_OK            # nothing to move
    assert gk(4, 128, 7, 2) == _lib.PH_ERR_ARG       # x does not divide the head size
    assert gk(4, 128, 8, 3) == _lib.PH_ERR_DTYPE
    assert gk(4, 128, 8, 2, idx=5) == _lib.PH_ERR_ARG
    gv = lambda n, bs: lib.ph_gather_blocked_v(None, None, None, None, 0, n, 2, 128, bs, 2, 4096, 2048, 16, 1, 256, 128,
                                               1, None)
    assert gv(4, 16) == _lib.PH_ERR_ARG and gv(0, 16) == _lib.PH_OK and gv(4, 0) == _lib.PH_ERR_ARG
    assert lib.ph_suffix_plan_build(None, 4, 512, 256, None, None, None, None) == _lib.PH_ERR_ARG      # null pointers
    assert lib.ph_suffix_plan_build(None, 0, 512, 256, None, None, None, None) == _lib.PH_OK           # no requests
    assert lib.ph_suffix_plan_build(None, 8193, 512, 256, None, None, None, None) == _lib.PH_ERR_ARG   # beyond the device planner
    assert lib.ph_suffix_plan_build(None, 4, 512, 0, None, None, None, None) == _lib.PH_ERR_ARG
    assert lib.ph_suffix_plan_build(None, 4, -1, 256, None, None, None, None) == _lib.PH_ERR_ARG       # negative bound
    assert lib.ph_sample_top_p(None, 32000, None, None, None, None, 4, 32000, 0, None) == _lib.PH_ERR_ARG  # null pointers
    assert lib.ph_sample_top_p(None, 32000, None, None, None, None, 0, 32000, 2, None) == _lib.PH_OK       # no rows
    assert lib.ph_sample_top_p(None, 32000, None, None, None, None, 4, 32000, 7, None) == _lib.PH_ERR_DTYPE
    assert lib.ph_sample_top_p(None, 100, None, None, None, None, 4, 32000, 0, None) == _lib.PH_ERR_ARG    # rows overlap
    assert lib.ph_sample_top_p(None, 0, None, None, None, None, 4, 0, 0, None) == _lib.PH_ERR_ARG
    assert lib.ph_suffix_tables_append(None, 64, None, None, None, -1, None) == _lib.PH_ERR_ARG
    assert lib.ph_suffix_tables_append(None, 64, None, None, None, 0, None) == _lib.PH_OK
    assert lib.ph_suffix_tables_append(None, 64, None, None, None, 3, None) == _lib.PH_ERR_ARG


def test_static_scratch_entry_point_refuses_oversize_without_a_gpu():
    """The size check of ph_decode_attention_static comes before anything touches the device."""
    from parrotserve_amd import _lib

    lib = _lib.load()
    assert lib.ph_decode_static_scratch_bytes() == 32 << 20
    assert lib.ph_decode_workspace_bytes(64, 32, 128, 1, 4096, 512, 0, 320) < lib.ph_decode_static_scratch_bytes()
    rc = lib.ph_decode_attention_static(1, 1, 1, 1, 4096, 32, 128, 0, 4096, 4096, 4096, 1.0, 0, None, None, None, None,
                                        0, 1, None, 8192, 4096 * 8192, 1, 8192, 32, None, None)
    assert rc == _lib.PH_ERR_SCRATCH and "scratch" in _lib.status_string(rc)


def test_cpu_tensors_are_refused_loudly():
    import torch

    from parrotserve_amd import kernels

    x = torch.zeros(4, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU only"):
        kernels.vllm_rms_norm(x, torch.ones(64, dtype=torch.float16), 1e-6)
