"""Host-side checks of the scratch-memory contract that need no GPU: the workspace-size queries
are plain host arithmetic (they run an entry point's own choice of kernels with the launches
switched off), and a *_ws call whose workspace is missing fails before anything is launched."""
import ctypes

from repdl_amd import _lib

P = ctypes.c_void_p
ALIGNED, OFF = P(0x7F0000000000), P(0x7F0000000004)

# (N, IC, H, W, OC, KH, KW, sH, sW, pH, pW)
LAYERS = [
    (64, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1),
    (64, 256, 56, 56, 64, 1, 1, 1, 1, 0, 0),
    (64, 64, 56, 56, 128, 3, 3, 2, 2, 1, 1),
    (64, 512, 7, 7, 512, 3, 3, 1, 1, 1, 1),
    (16, 3, 224, 224, 64, 7, 7, 2, 2, 3, 3),
    (2, 5, 11, 12, 9, 2, 3, 1, 1, 0, 1),
]


def _queries(layer, a, b):
    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW = layer
    OH, OW = (H + 2 * pH - KH) // sH + 1, (W + 2 * pW - KW) // sW + 1
    lib = _lib.lib()
    return (lib.repdl_hip_conv2d_workspace_bytes(a, b, N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, 1),
            lib.repdl_hip_conv2d_grad_input_workspace_bytes(a, b, N, OC, OH, OW, IC, KH, KW, H, W, sH, sW, pH, pW),
            lib.repdl_hip_conv2d_grad_kernel_workspace_bytes(a, b, N, IC, H, W, OC, OH, OW, KH, KW, sH, sW, pH, pW))


def test_queries_run_without_a_device_and_bound_any_alignment():
    for layer in LAYERS:
        known = _queries(layer, ALIGNED, ALIGNED)
        anyp = _queries(layer, None, None)
        for k, a in zip(known, anyp):
            assert 0 <= k <= a < (1 << 36), (layer, known, anyp)  # NULL pointers: a bound for every alignment
        for mixed in (_queries(layer, OFF, ALIGNED), _queries(layer, ALIGNED, OFF), _queries(layer, OFF, OFF)):
            assert all(m <= a for m, a in zip(mixed, anyp)), layer
        assert _queries(layer, ALIGNED, ALIGNED) == known  # no state is kept between queries


def test_queries_of_the_sums_and_the_loss():
    lib = _lib.lib()
    assert lib.repdl_hip_sum2d_dim1_workspace_bytes(16384, 16384) == 0  # many rows: one lane per chain, no scratch
    few = lib.repdl_hip_sum2d_dim1_workspace_bytes(16, 802816)
    assert few > 0 and lib.repdl_hip_sum2d_dim1_workspace_bytes(32, 802816) > few
    assert lib.repdl_hip_sum4d_dim023_workspace_bytes(64, 64, 56, 56) > 0
    assert lib.repdl_hip_sum4d_dim023_workspace_bytes(64, 64, 7, 7) == 0
    assert lib.repdl_hip_cross_entropy_workspace_bytes(0, 10) == 0
    small, large = lib.repdl_hip_cross_entropy_workspace_bytes(64, 10), lib.repdl_hip_cross_entropy_workspace_bytes(65536, 1000)
    assert 64 * 4 <= small <= 4096
    assert large >= 65536 * 4 + lib.repdl_hip_sum1d_workspace_bytes(65536)


def test_invalid_arguments_need_no_workspace():
    lib = _lib.lib()
    assert lib.repdl_hip_conv2d_workspace_bytes(ALIGNED, ALIGNED, 1, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 2) == 0  # groups do not divide
    assert lib.repdl_hip_conv2d_workspace_bytes(ALIGNED, ALIGNED, 1, 4, 2, 2, 4, 3, 3, 1, 1, 0, 0, 1) == 0  # kernel larger than the input
    assert lib.repdl_hip_sum2d_dim1_workspace_bytes(-1, 5) == 0


def test_missing_workspace_is_refused_before_any_launch():
    """No device here: a call that got as far as a launch would report a runtime error, not this code."""
    lib = _lib.lib()
    N, IC, H, W, OC, KH, KW, sH, sW, pH, pW = LAYERS[0]
    assert lib.repdl_hip_conv2d_workspace_bytes(ALIGNED, ALIGNED, N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, 1) > 0
    rc = lib.repdl_hip_conv2d_ws(ALIGNED, ALIGNED, None, ALIGNED, N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, 1, None, 0, None)
    assert rc == -3 and b"workspace" in lib.repdl_hip_error_string(rc)
    rc = lib.repdl_hip_sum4d_dim023_ws(ALIGNED, ALIGNED, 64, 64, 56, 56, 0, ALIGNED, 1024, None)
    assert rc == -3
    rc = lib.repdl_hip_cross_entropy_ws(ALIGNED, ALIGNED, ALIGNED, 64, 10, None, 0, None)
    assert rc == -3
