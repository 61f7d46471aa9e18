"""The C-ABI library loads and exports every symbol include/mcn_hip.h declares (no compute calls: this
runs without a GPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mcn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"MCN_API\s+[\w\s\*]+?\b(mcn_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    syms = declared_symbols()
    for must in ("mcn_conv_backward_data", "mcn_conv_backward_filter", "mcn_conv_backward_bias", "mcn_conv_forward",
                 "mcn_bnorm_backward", "mcn_bnorm_forward", "mcn_pool_backward", "mcn_pool_forward"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    from matconvnet_amd import capi
    lib = ctypes.CDLL(capi.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing
    # and the binding knows a prototype for each of them
    assert sorted(capi.PROTOTYPES) == declared_symbols()


def test_host_side_validation_needs_no_gpu():
    """Shape validation happens on the host before any launch."""
    from matconvnet_amd import capi
    g = capi.conv_geom((56, 56, 256, 64), (3, 3, 256, 256), 1, 1, 1)
    assert capi.conv_out_shape(g) == (56, 56, 256, 64)
    p = capi.pool_geom((112, 112, 64, 32), 3, 2, 1, "max")
    assert capi.pool_out_shape(p) == (56, 56, 64, 32)
    assert capi.lib().mcn_error_name(capi.ILLEGAL_ARGUMENT) == b"illegal argument error"
    try:
        capi.pool_out_shape(capi.pool_geom((4, 4, 1, 1), 3, 0, 0, "max"))
        raise AssertionError("stride 0 accepted")
    except capi.McnError as e:
        assert e.code == capi.ILLEGAL_ARGUMENT and "STRIDE" in e.message


def test_marking_streams_as_running_beside_another_is_host_bookkeeping():
    """mcn_stream_beside keeps a table of at most 16 stream handles (no GPU call): the null stream is refused, marking
    twice and unmarking an unmarked handle are harmless, the seventeenth distinct handle is refused until one is freed."""
    import ctypes as C
    from matconvnet_amd import capi
    L = capi.lib()
    handles = [C.c_void_p(0x1000 + 16 * i) for i in range(17)]  # (stand-ins: the table only compares handles)
    try:
        assert L.mcn_stream_beside(None, 1) == capi.ILLEGAL_ARGUMENT
        for h in handles[:16]:
            assert L.mcn_stream_beside(h, 1) == 0
        assert L.mcn_stream_beside(handles[3], 1) == 0          # already marked
        assert L.mcn_stream_beside(handles[16], 1) != 0         # table full
        assert L.mcn_stream_beside(handles[5], 0) == 0
        assert L.mcn_stream_beside(handles[16], 1) == 0         # a slot is free again
        assert L.mcn_stream_beside(handles[5], 0) == 0          # not marked: nothing to do
    finally:
        for h in handles:
            L.mcn_stream_beside(h, 0)
