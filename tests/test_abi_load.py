"""CPU-side checks of the drop-in boundary: the shared library loads without a GPU, exports every
symbol the public header declares, and reports errors instead of computing without a device."""
import ctypes as C

import pytest

from warpdecode_amd import capi, synth


def test_exports_every_declared_symbol():
    lib = capi.load()
    declared = capi.declared_symbols()
    assert len(declared) >= 40
    missing = [s for s in declared if not hasattr(lib, s)]
    assert not missing, missing


@pytest.mark.parametrize("t", [synth.Q4_0, synth.Q8_0, synth.IQ4_NL, synth.IQ3_S, synth.IQ2_S])
def test_block_geometry(t):
    lib = capi.load()
    assert lib.wd_row_bytes(t, 2048) == synth.row_bytes(t, 2048)
    assert lib.wd_row_bytes(t, 2048 + 1) == 0
    assert lib.wd_tensor_bytes(t, 512, 2048) == 512 * synth.row_bytes(t, 2048)
    assert lib.wd_row_bytes(99, 2048) == 0


def test_argument_errors_are_reported():
    lib = capi.load()
    # geometry is validated before any device work, so these fail the same way with or without a GPU
    assert lib.wd_q8_k_quantize_f32(None, 100, None, None, None, None) == -1
    assert b"multiple of 256" in lib.wd_last_error()
    assert lib.wd_topk_softmax(None, 12, 2, 1.0, None, None, None) == -1
    assert b"multiple of 8" in lib.wd_last_error()
    assert lib.wd_gemv_q8_k_f32(synth.Q8_0, C.c_void_p(8), 4, 256, None, None, None, None, None) == -1
    with pytest.raises(capi.WdError):
        capi.call("wd_q8_0_quantize_f32", None, 33, None, None, None)


def test_profiler_switched_off_touches_nothing():
    """The site profiler's names follow the reference's numbering (src/qwen38_moe.cuh:296-352), and with the switch off
    its hooks are no-ops that need no device."""
    from warpdecode_amd import capi
    lib = capi.load()
    names = [lib.wd_profile_site_name(i).decode() for i in range(24)]
    assert names[0] == "moe.stage_total" and names[1] == "moe.routed_total" and names[2] == "moe.router_select"
    assert names[10] == "moe.acquire" and names[13] == "moe.batch.gate_up" and names[17] == "moe.batch.accum"
    assert names[20] == "moe.finish" and names[23] == "moe.mirror" and len(set(names)) == 24
    assert lib.wd_profile_site_name(24) == b"moe.fused.ab"
    assert lib.wd_profile_site_name(-1) == b"unknown" and lib.wd_profile_site_name(1000) == b"unknown"
    assert lib.wd_profile_enabled() == 0
    capi.call("wd_profile_begin", 0, None)
    capi.call("wd_profile_end", 0, None)
    capi.call("wd_profile_flush_token")
    st, tokens = capi.ProfileSiteStat(), C.c_ulonglong(7)
    capi.call("wd_profile_site", 0, C.byref(st), C.byref(tokens))
    assert (st.calls, st.recorded, st.dropped, st.host_ms, tokens.value) == (0, 0, 0, 0.0, 0)
    assert lib.wd_profile_begin(1000, None) != 0 and b"out of range" in lib.wd_last_error()
    need = lib.wd_profile_report(None, 0)
    buf = C.create_string_buffer(need + 1)
    assert lib.wd_profile_report(buf, need + 1) == need
    assert buf.value == b"[moe-profile] tokens=0 unit=ms_per_token\n"
