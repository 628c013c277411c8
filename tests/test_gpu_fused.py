"""GPU: the cooperative launch of the shift convolution -- tiles shared between workgroups finished by
the last arrival through partial tiles in the workspace -- and its fused epilogue
(ds_conv2d_tiled_fused_i32), through the C ABI, bit for bit against the oracle chain."""
import ctypes

import numpy as np
import pytest
import torch

from deepshift_amd import _lib, kernels
from oracle import shift_oracle as so
from tests.conftest import Tune, random_activations, random_codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NTHREADS = 8
U = _lib.DS_BITS_TOP_UNUSED


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _stream():
    return _lib.current_stream(torch.device(DEV))


def abi_conv_tiled(xp, blob, bias, O, FH, FW, stride, bits, with_workspace=True):
    Nb, C, Hp, Wp = xp.shape
    sh, sw = stride
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_tiled_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits) if with_workspace else 0
    ws = torch.full((max(ws_bytes, 1),), 0x77, dtype=torch.uint8, device=DEV)   # stale contents on purpose
    total, guard = Nb * O * OH * OW, 64
    ybuf = torch.full((total + 2 * guard,), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    y = ybuf[guard:guard + total]
    xd = _dev(xp)
    bd = None if bias is None else _dev(bias)
    _lib.call("ds_conv2d_tiled_i32", _lib.ptr(xd), _lib.ptr(blob), _lib.ptr(bd), ctypes.c_void_p(y.data_ptr()),
              Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits, 0, _lib.ptr(ws) if ws_bytes else None, ws_bytes, _stream())
    torch.cuda.synchronize()
    host = ybuf.cpu().numpy()
    assert (host[:guard] == 0x5A5A5A5A).all() and (host[guard + total:] == 0x5A5A5A5A).all()
    return host[guard:guard + total].reshape(Nb, O, OH, OW)


def abi_conv_fused(xp, blob, bias, O, FH, FW, stride, bits, F_in, scale, shift, res, relu, want_float, emit):
    """emit = (ph, pw, I, F, torch dtype) or None; returns (out or None, q or None), guard bands checked."""
    Nb, C, Hp, Wp = xp.shape
    sh, sw = stride
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_tiled_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits)
    # the 64-channel form (fields of at most 4 bits) needs the workspace, other layers none
    assert ws_bytes > 0 or O % 64 != 0 or (bits & 0xff) > 4
    ws = torch.full((max(ws_bytes, 1),), 0x77, dtype=torch.uint8, device=DEV)
    guard = 64
    n_out = Nb * O * OH * OW
    obuf = torch.full((n_out + 2 * guard,), 12345.0, dtype=torch.float32, device=DEV)
    out = obuf[guard:guard + n_out] if want_float else None
    q = qbuf = None
    ph = pw = 0
    I, Fq, qb = 16, 16, 4
    if emit is not None:
        ph, pw, I, Fq, dtype = emit
        n_q = Nb * O * (OH + 2 * ph) * (OW + 2 * pw)
        qbuf = torch.full((n_q + 2 * guard,), 0x5A, dtype=dtype, device=DEV)
        q = qbuf[guard:guard + n_q]
        qb = 1 if dtype == torch.int8 else 4
    xd = _dev(xp)
    t = [None if a is None else _dev(a) for a in (bias, scale, shift, res)]
    _lib.call("ds_conv2d_tiled_fused_i32", _lib.ptr(xd), _lib.ptr(blob), _lib.ptr(t[0]),
              None if out is None else ctypes.c_void_p(out.data_ptr()),
              None if q is None else ctypes.c_void_p(q.data_ptr()), _lib.ptr(t[1]), _lib.ptr(t[2]), _lib.ptr(t[3]),
              Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits, 0, F_in, int(relu), I, Fq, ph, pw, qb,
              _lib.ptr(ws) if ws_bytes else None, ws_bytes, _stream())
    torch.cuda.synchronize()
    oh = obuf.cpu().numpy()
    assert (oh[:guard] == 12345.0).all() and (oh[guard + n_out:] == 12345.0).all(), "write outside out"
    got_out = oh[guard:guard + n_out].reshape(Nb, O, OH, OW) if want_float else None
    if not want_float:
        assert (oh == 12345.0).all()
    got_q = None
    if q is not None:
        qh = qbuf.cpu().numpy()
        assert (qh[:guard] == 0x5A).all() and (qh[guard + n_q:] == 0x5A).all(), "write outside q"
        got_q = qh[guard:guard + n_q].reshape(Nb, O, OH + 2 * ph, OW + 2 * pw).astype(np.int32)
    return got_out, got_q


# geometries: many tiles per workgroup, tiles shared by several workgroups (few pixels, long reduction),
# ragged pixel counts, strides, 1x1 and 3x3, several channel tiles
GEOMS = [
    # Nb, C, Hp, Wp, O, FH, FW, stride
    (2, 64, 30, 30, 64, 3, 3, (1, 1)),       # 1568 pixels: 13 tiles, K = 576
    (1, 256, 9, 9, 128, 3, 3, (1, 1)),       # 49 pixels: one ragged pixel tile, every tile cut many times
    (3, 128, 16, 15, 192, 3, 3, (2, 2)),     # strided, three channel tiles
    (5, 384, 12, 12, 64, 1, 1, (1, 1)),      # 1x1 with a long reduction (64 K groups)
    (2, 40, 21, 19, 64, 5, 3, (1, 2)),       # 5x3 filter, K = 600
    # short reductions on the 64-channel form: the 1x1 convolutions of a bottleneck block (modules.py:312-340
    # followed by the same glue as every other layer)
    (4, 64, 20, 20, 256, 1, 1, (1, 1)),      # 64 -> 256, 11 K groups: less than a group per wave of some tiles
    (3, 256, 14, 14, 64, 1, 1, (1, 1)),      # 256 -> 64, 43 K groups
    (2, 256, 17, 16, 512, 1, 1, (2, 2)),     # strided shortcut, eight channel tiles
    (6, 3, 37, 37, 64, 7, 7, (2, 2)),        # a stem without its pooling: K = 147, a partial last group
    # 100 pixel tiles on 32 workgroups: three tiles and a bit per share, so the share space walks the first 96
    # tiles transposed (index j at tile (j mod 3) * 32 + j / 3) and the last four as they lie
    (8, 64, 40, 40, 64, 1, 1, (1, 1)),
]
# layers that are not a multiple of 64 channels wide: the fused form of the two-instruction kernel
NARROW_GEOMS = [
    (3, 16, 34, 34, 16, 3, 3, (1, 1)),       # ResNet-20's first stage
    (2, 16, 34, 33, 32, 3, 3, (2, 2)),       # strided, 32 channels, ragged pixel count
    (2, 7, 11, 13, 40, 3, 2, (1, 1)),        # 40 channels: a partial channel tile, K = 42
    (5, 32, 10, 10, 10, 1, 1, (1, 1)),       # 1x1, fewer channels than a tile holds
    (16, 32, 65, 65, 64, 3, 3, (2, 2)),      # 64 channels but only 48 K groups: this kernel, not the 64-channel form
    (128, 3, 34, 34, 16, 3, 3, (1, 1)),      # a first convolution, K = 27: one or two K groups per wave
]


@pytest.mark.parametrize("geom", GEOMS, ids=lambda g: "x".join(str(v) for v in g[:7]))
@pytest.mark.parametrize("bits", [4, 2])
def test_cooperative_launch_matches_oracle(oracle, rng, geom, bits):
    """ds_conv2d_tiled_i32 with its workspace (cooperative launch, forced where the dispatch would pick
    another one) and without it (per-wave shares), both flag forms, over stale workspace contents."""
    Nb, C, Hp, Wp, O, FH, FW, stride = geom
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    top = 2 ** bits - 2
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=top)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32)
    want = oracle.conv2d(xp, -s, sign, bias, stride, nthreads=NTHREADS)
    blob = kernels.tile_weights(_dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)).reshape(-1),
                                O, C, FH, FW, bits, 0)
    with Tune(planes=1, split=0, cu=4):
        for b in (bits, bits | U):
            np.testing.assert_array_equal(abi_conv_tiled(xp, blob, bias, O, FH, FW, stride, b), want)
        np.testing.assert_array_equal(abi_conv_tiled(xp, blob, None, O, FH, FW, stride, bits),
                                      oracle.conv2d(xp, -s, sign, None, stride, nthreads=NTHREADS))
        np.testing.assert_array_equal(abi_conv_tiled(xp, blob, bias, O, FH, FW, stride, bits, False), want)


def test_many_short_tiles_run_in_whole_tile_shares(oracle, rng):
    """A short reduction over many pixel tiles (a 7x7 stem's shape class): the cooperative launch hands
    out whole tiles, one per wave in rounds of four, the rest of a share split over its waves.  4616
    tiles on 512 workgroups leave shares of 9 and 10 tiles: both paths run, and the last tile is ragged."""
    Nb, C, Hp, Wp, O, FH, FW, stride = 2, 3, 550, 549, 64, 7, 7, (1, 1)
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=14)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32)
    want = oracle.conv2d(xp, -s, sign, bias, stride, nthreads=NTHREADS)
    blob = kernels.tile_weights(_dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), 4)).reshape(-1),
                                O, C, FH, FW, 4, 0)
    for b in (4, 4 | U):
        np.testing.assert_array_equal(abi_conv_tiled(xp, blob, bias, O, FH, FW, stride, b), want)


def test_cooperative_launch_replays_in_a_graph(oracle, rng):
    """A captured launch keeps its arguments, the counters' tag among them: every replay must find the
    arrival counters as a finished launch leaves them.  Replays alternate with eager launches on the
    same workspace and are checked against the oracle each time."""
    Nb, C, Hp, Wp, O, FH, FW, stride = 1, 256, 9, 9, 128, 3, 3, (1, 1)   # every tile cut many times
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=14)
    blob = kernels.tile_weights(_dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), 4)).reshape(-1),
                                O, C, FH, FW, 4, 0)
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_tiled_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, 1, 1, 4)
    ws = torch.full((ws_bytes,), 0x77, dtype=torch.uint8, device=DEV)
    xd = torch.zeros((Nb, C, Hp, Wp), dtype=torch.int32, device=DEV)
    y = torch.zeros((Nb, O, Hp - 2, Wp - 2), dtype=torch.int32, device=DEV)

    def launch():
        _lib.call("ds_conv2d_tiled_i32", _lib.ptr(xd), _lib.ptr(blob), None, _lib.ptr(y), Nb, C, Hp, Wp, O, FH, FW,
                  1, 1, 4, 0, _lib.ptr(ws), ws_bytes, _stream())

    with Tune(planes=1, split=0, cu=4):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            launch()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            launch()
        for step in range(4):
            xp = random_activations(rng, (Nb, C, Hp, Wp))
            want = oracle.conv2d(xp, -s, sign, None, stride, nthreads=NTHREADS)
            xd.copy_(_dev(xp))
            y.fill_(-1)
            graph.replay()
            torch.cuda.synchronize()
            np.testing.assert_array_equal(y.cpu().numpy(), want, err_msg="replay %d" % step)
            y.fill_(-1)
            launch()
            torch.cuda.synchronize()
            np.testing.assert_array_equal(y.cpu().numpy(), want, err_msg="eager after replay %d" % step)


@pytest.mark.parametrize("geom", GEOMS + NARROW_GEOMS, ids=lambda g: "x".join(str(v) for v in g[:7]))
def test_fused_epilogue_matches_oracle_chain(oracle, rng, geom):
    """Float and fixed-point outputs of the fused call against oracle.conv2d -> np_dequantize_affine ->
    np_requantize, for every combination of what may follow the layer."""
    Nb, C, Hp, Wp, O, FH, FW, stride = geom
    OH, OW = (Hp - FH) // stride[0] + 1, (Wp - FW) // stride[1] + 1
    xp = rng.integers(-2 ** 17, 2 ** 19, size=(Nb, C, Hp, Wp)).astype(np.int32)
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=14)
    bias = rng.integers(-2 ** 16, 2 ** 16, size=O).astype(np.int32)
    y = oracle.conv2d(xp, -s, sign, bias, stride, nthreads=NTHREADS)
    blob = kernels.tile_weights(_dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), 4)).reshape(-1),
                                O, C, FH, FW, 4, 0)
    scale = ((rng.random(O) + 0.5) * 2.0 ** -6).astype(np.float32)
    shift = rng.standard_normal(O).astype(np.float32)
    res = (rng.standard_normal((Nb, O, OH, OW)) * 2).astype(np.float32)
    cases = [
        (scale, shift, res, True, True, (1, 1, 16, 16, torch.int32)),     # block end: float + q
        (scale, shift, None, True, False, (1, 1, 16, 16, torch.int32)),   # between two convolutions: q only
        (scale, None, None, False, True, None),                           # float only
        (None, None, None, False, True, (0, 0, 16, 16, torch.int32)),     # plain dequantisation, no padding
        (scale, shift, res, True, True, (2, 3, 12, 4, torch.int32)),      # wider padding, another format
        (scale, shift, None, True, False, (1, 1, 3, 5, torch.int8)),      # int8 consumer
    ]
    for sc, sh, r, relu, want_float, emit in cases:
        v = so.np_dequantize_affine(y, 16, sc, sh, r, relu)
        out, q = abi_conv_fused(xp, blob, bias, O, FH, FW, stride, 4 | U, 16, sc, sh, r, relu, want_float, emit)
        if want_float:
            np.testing.assert_array_equal(out, v)
        if emit is not None:
            np.testing.assert_array_equal(q, so.np_requantize(v, emit[2], emit[3], emit[:2]))


# layers of 32, 96 ... channels: the shift-plane loop inside the one-tile-per-workgroup launch (two pixel rows x
# 32 channels per lane), every form of it
PLANE32_CASES = [
    # Nb, C, Hp, Wp, O, FH, FW, stride, bits, top value unused
    (3, 16, 34, 33, 32, 3, 3, (2, 2), 4, True),     # K = 144: whole groups, the form without the top plane
    (3, 16, 18, 18, 32, 3, 3, (1, 1), 4, False),    # shifts up to 15: every plane
    (2, 7, 25, 23, 96, 3, 3, (1, 1), 4, True),      # K = 63: a partial last group, top plane held at zero
    (2, 7, 25, 23, 32, 3, 3, (1, 1), 4, False),     # ... decoded by the scalar tail
    (4, 32, 18, 18, 32, 3, 3, (1, 1), 4, True),     # ResNet-20's second stage in small
    (2, 40, 14, 15, 64 + 32, 3, 3, (1, 1), 3, True),   # 3-bit fields, 8 codes per word
    (2, 40, 14, 15, 32, 3, 3, (1, 1), 2, False),    # 2-bit fields, 10 codes per word
    (2, 150, 12, 12, 32, 1, 1, (1, 1), 1, False),   # 1-bit fields, 16 codes per word: K = 150 leaves a partial group
    (1, 24, 9, 9, 160, 3, 3, (1, 1), 4, True),      # 49 pixels: one ragged tile, five channel tiles
]


@pytest.mark.parametrize("case", PLANE32_CASES, ids=lambda c: "x".join(str(v) for v in c[:7]) + "-b%d%s" % (c[8], "u" if c[9] else ""))
def test_narrow_plane_form_matches_oracle_chain(oracle, rng, case):
    """The fused launch of layers whose channel count is a multiple of 32 but not of 64 against the oracle
    chain, and against the two-instruction loop it replaces (forced through the test hook)."""
    Nb, C, Hp, Wp, O, FH, FW, stride, bits, unused = case
    OH, OW = (Hp - FH) // stride[0] + 1, (Wp - FW) // stride[1] + 1
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=2 ** bits - (2 if unused else 1))
    bias = rng.integers(-2 ** 16, 2 ** 16, size=O).astype(np.int32)
    y = oracle.conv2d(xp, -s, sign, bias, stride, nthreads=NTHREADS)
    blob = kernels.tile_weights(_dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)).reshape(-1),
                                O, C, FH, FW, bits, 0)
    scale = ((rng.random(O) + 0.5) * 2.0 ** -6).astype(np.float32)
    shift = rng.standard_normal(O).astype(np.float32)
    res = (rng.standard_normal((Nb, O, OH, OW)) * 2).astype(np.float32)
    flag = bits | (U if unused else 0)
    for sc, sh, r, relu, want_float, emit in [
        (scale, shift, res, True, True, (1, 1, 16, 16, torch.int32)),
        (None, None, None, False, True, None),
        (scale, shift, None, True, False, (1, 2, 3, 5, torch.int8)),
    ]:
        v = so.np_dequantize_affine(y, 16, sc, sh, r, relu)
        out, q = abi_conv_fused(xp, blob, bias, O, FH, FW, stride, flag, 16, sc, sh, r, relu, want_float, emit)
        with Tune(planes=0):
            out2, q2 = abi_conv_fused(xp, blob, bias, O, FH, FW, stride, flag, 16, sc, sh, r, relu, want_float, emit)
        if want_float:
            np.testing.assert_array_equal(out, v)
            np.testing.assert_array_equal(out2, v)
        if emit is not None:
            want_q = so.np_requantize(v, emit[2], emit[3], emit[:2])
            np.testing.assert_array_equal(q, want_q)
            np.testing.assert_array_equal(q2, want_q)


@pytest.mark.parametrize("geom", [GEOMS[0], NARROW_GEOMS[0], NARROW_GEOMS[1]], ids=["64-channel", "16-channel", "32-channel"])
def test_fused_round_to_fixed_saturates(oracle, rng, geom):
    """Values beyond the fixed-point range clamp to its ends (utils.py:7-21), infinities included, and a NaN
    (a broken BatchNorm constant) becomes 0 as in the conversion kernels: the epilogue converts with the
    hardware's saturating floor conversion and clamps on integers."""
    Nb, C, Hp, Wp, O, FH, FW, stride = geom
    xp = rng.integers(-2 ** 17, 2 ** 19, size=(Nb, C, Hp, Wp)).astype(np.int32)
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=14)
    y = oracle.conv2d(xp, -s, sign, None, stride, nthreads=NTHREADS)
    blob = kernels.tile_weights(_dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), 4)).reshape(-1),
                                O, C, FH, FW, 4, 0)
    scale = (rng.choice([1e-3, 1.0, 3e4, 1e9], size=O) * rng.choice([-1.0, 1.0], size=O)).astype(np.float32)
    shift = rng.standard_normal(O).astype(np.float32)
    shift[1], shift[2], shift[3] = np.inf, -np.inf, np.nan
    for I, F, dtype in ((16, 16, torch.int32), (12, 4, torch.int32), (3, 5, torch.int8)):
        out, q = abi_conv_fused(xp, blob, None, O, FH, FW, stride, 4 | U, 16, scale, shift, None, False, True,
                                (1, 1, I, F, dtype))
        with np.errstate(invalid="ignore", over="ignore"):
            v = so.np_dequantize_affine(y, 16, scale, shift, None, False)
            finite = v.copy()
            finite[:, 3] = 0.0
            want = so.np_requantize(finite, I, F, (1, 1))
        np.testing.assert_array_equal(out[:, :3], v[:, :3])
        np.testing.assert_array_equal(out[:, 4:], v[:, 4:])
        assert np.isnan(out[:, 3]).all()
        np.testing.assert_array_equal(q, want)
        hi, lo = (2 ** (I - 1) - 1) * 2 ** F, -2 ** (I - 1 + F)
        assert (q[:, 1, 1:-1, 1:-1] == hi).all() and (q[:, 2, 1:-1, 1:-1] == lo).all() and (q[:, 3] == 0).all()
        assert (q == hi).sum() > q[:, 1, 1:-1, 1:-1].size and (q == lo).sum() > q[:, 2, 1:-1, 1:-1].size


def test_border_kept_writes_the_interior_only(oracle, rng):
    """q_bytes | DS_Q_BORDER_KEPT: the caller's buffer keeps its padding (zeroed once by the caller), the
    kernel overwrites the interior; with the flag off the kernel writes the padding itself."""
    Nb, C, Hp, Wp, O, FH, FW, stride = GEOMS[0]
    OH, OW = Hp - 2, Wp - 2
    xp = rng.integers(-2 ** 17, 2 ** 19, size=(Nb, C, Hp, Wp)).astype(np.int32)
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=14)
    y = oracle.conv2d(xp, -s, sign, None, stride, nthreads=NTHREADS)
    want = so.np_requantize(so.np_dequantize_affine(y, 16, None, None, None, True), 16, 16, (1, 2))
    blob = kernels.tile_weights(_dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), 4)).reshape(-1),
                                O, C, FH, FW, 4, 0)
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_tiled_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, 1, 1, 4)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    xd = _dev(xp)
    for kept in (True, False):
        q = torch.full((Nb, O, OH + 2, OW + 4), 7, dtype=torch.int32, device=DEV)
        _lib.call("ds_conv2d_tiled_fused_i32", _lib.ptr(xd), _lib.ptr(blob), None, None, _lib.ptr(q), None, None,
                  None, Nb, C, Hp, Wp, O, FH, FW, 1, 1, 4, 0, 16, 1, 16, 16, 1, 2,
                  4 | (_lib.DS_Q_BORDER_KEPT if kept else 0), _lib.ptr(ws), ws_bytes, _stream())
        got = q.cpu().numpy()
        np.testing.assert_array_equal(got[:, :, 1:-1, 2:-2], want[:, :, 1:-1, 2:-2])
        border = np.ones_like(got, bool)
        border[:, :, 1:-1, 2:-2] = False
        assert (got[border] == (7 if kept else 0)).all()


def test_fused_entry_point_refuses_what_it_cannot_do(rng):
    L = _lib.lib()
    one = ctypes.c_void_p(256)
    args = lambda O, bits, base, ws: (one, one, None, one, None, None, None, None, 2, 64, 30, 30, O, 3, 3, 1, 1,
                                      bits, base, 16, 0, 16, 16, 0, 0, 4, one if ws else None, 1 << 30 if ws else 0,
                                      None)
    Z = _lib.DS_BITS_ZERO_TOP
    assert L.ds_conv2d_tiled_fused_i32(*args(48, 6, 0, True)) == -1     # 6-bit (general) codes
    assert L.ds_conv2d_tiled_fused_i32(*args(48, 4 | Z, 0, True)) == -1  # zero-top blob on a narrow layer
    assert L.ds_conv2d_tiled_fused_i32(*args(64, 4, -1, True)) == -1    # left shifts
    assert L.ds_conv2d_tiled_fused_i32(*args(64, 4, 0, False)) == -4    # 64-channel form without its workspace
    assert L.ds_conv2d_tiled_fusable(64, 64, 58, 58, 64, 3, 3, 1, 1, 4 | U, 0) == 1
    assert L.ds_conv2d_tiled_fusable(64, 64, 56, 56, 128, 1, 1, 2, 2, 4, 0) == 1   # short reduction, 64-channel form
    # layers the two-instruction kernel serves: fused there when single pixel rows fill the machine
    assert L.ds_conv2d_tiled_fusable(64, 64, 58, 58, 64, 3, 3, 1, 1, 5, 0) == 1
    assert L.ds_conv2d_tiled_fusable(64, 64, 58, 58, 48, 3, 3, 1, 1, 4, 0) == 1
    assert L.ds_conv2d_tiled_fusable(256, 16, 34, 34, 16, 3, 3, 1, 1, 4 | U, 0) == 1
    assert L.ds_conv2d_tiled_fusable(1, 16, 34, 34, 16, 3, 3, 1, 1, 4, 0) == 0     # 16 waves of pixels
    assert L.ds_conv2d_tiled_fusable(64, 64, 58, 58, 48, 3, 3, 1, 1, 6, 0) == 0
    assert L.ds_conv2d_tiled_fusable(64, 64, 58, 58, 48, 3, 3, 1, 1, 4, -2) == 0


def test_fused_module_path_equals_the_separate_passes():
    """conv_kernel_forward with the fused epilogue against the same call with it switched off (int32 sums,
    then the conversion pass): every output bit-identical."""
    from deepshift_amd import modules
    torch.manual_seed(3)
    conv = modules.Conv2dShift(64, 128, 3, stride=1, padding=1, use_kernel=True).to(DEV)
    conv.sign.data = torch.where(conv.sign.data >= 0, torch.ones_like(conv.sign), -torch.ones_like(conv.sign))
    x = torch.randn(16, 64, 40, 40, device=DEV)
    scale = torch.rand(128, device=DEV) + 0.5
    shift = torch.randn(128, device=DEV)
    res = torch.randn(16, 128, 40, 40, device=DEV)
    cw = conv.packed_weights()
    assert kernels.conv2d_fusable((16, 64, 42, 42), 128, (3, 3), (1, 1), kernels.kernel_bits(cw), 0)
    results = {}

    def keep(r):  # the hand-off buffer is reused by the next call: copy what a call returned
        return tuple(t.clone() for t in (r if isinstance(r, tuple) else (r,)))

    for fused in (True, False):
        modules._FUSE_EPILOGUE = fused
        try:
            with torch.no_grad():
                results[fused] = [
                    keep(modules.conv_kernel_forward(conv, x, cw)),
                    keep(modules.conv_kernel_forward(conv, x, cw, scale, shift, res, True)),
                    keep(modules.conv_kernel_forward(conv, x, cw, scale, shift, res, True,
                                                     emit=((1, 1), 16, 16, True))),
                    keep(modules.conv_kernel_forward(conv, x, cw, scale, shift, None, True,
                                                     emit=((1, 1), 16, 16, False))),
                    # a second geometry replaces the cached buffer, a return to the first re-zeroes one
                    keep(modules.conv_kernel_forward(conv, x[:8], cw, scale, shift, None, True,
                                                     emit=((1, 1), 16, 16, False))),
                    keep(modules.conv_kernel_forward(conv, x, cw, scale, shift, None, True,
                                                     emit=((1, 1), 16, 16, False))),
                ]
        finally:
            modules._FUSE_EPILOGUE = True
    for a, b in zip(results[True], results[False]):
        a = a if isinstance(a, tuple) else (a,)
        b = b if isinstance(b, tuple) else (b,)
        for t, u in zip(a, b):
            assert torch.equal(t, u)


@pytest.mark.parametrize("geom", [
    # Nb, C, H, W, O_first, k, O_shortcut, stride
    (4, 64, 28, 28, 128, 3, 128, 2),     # a ResNet-18 down-sampling block in small
    (2, 128, 15, 13, 64, 3, 192, 2),     # odd sizes, different channel counts
    (3, 64, 12, 12, 64, 5, 64, 1),       # 5 x 5 first convolution (padding 2), stride 1
], ids=lambda g: "x".join(map(str, g)))
def test_pair_launch_matches_oracle_chain(oracle, rng, geom):
    """ds_conv2d_tiled_fused_pair_i32: a k x k convolution and a 1 x 1 shortcut over one padded input in one
    launch, each output against oracle.conv2d -> np_dequantize_affine -> np_requantize of the layer alone."""
    Nb, C, H, W, Oa, k, Ob, st = geom
    p = (k - 1) // 2
    x = rng.integers(-2 ** 17, 2 ** 19, size=(Nb, C, H, W)).astype(np.int32)
    xp = np.pad(x, ((0, 0), (0, 0), (p, p), (p, p)))
    sa, ga = random_codes(rng, (Oa, C, k, k), max_s=14)
    sb, gb = random_codes(rng, (Ob, C, 1, 1), max_s=14)
    ba = rng.integers(-2 ** 16, 2 ** 16, size=Oa).astype(np.int32)
    bb = rng.integers(-2 ** 16, 2 ** 16, size=Ob).astype(np.int32)
    ya = oracle.conv2d(xp, -sa, ga, ba, (st, st), nthreads=NTHREADS)
    yb = oracle.conv2d(x, -sb, gb, bb, (st, st), nthreads=NTHREADS)      # the shortcut sees the unpadded input
    assert ya.shape[2:] == yb.shape[2:]
    scale_a = ((rng.random(Oa) + 0.5) * 2.0 ** -6).astype(np.float32)
    shift_a = rng.standard_normal(Oa).astype(np.float32)
    scale_b = ((rng.random(Ob) + 0.5) * 2.0 ** -4).astype(np.float32)
    shift_b = rng.standard_normal(Ob).astype(np.float32)
    res_b = rng.standard_normal(yb.shape).astype(np.float32)
    blob_a = kernels.tile_weights(_dev(so.np_pack_words(sa.reshape(Oa, -1), ga.reshape(Oa, -1), 4)).reshape(-1),
                                  Oa, C, k, k, 4, 0)
    blob_b = kernels.tile_weights(_dev(so.np_pack_words(sb.reshape(Ob, -1), gb.reshape(Ob, -1), 4)).reshape(-1),
                                  Ob, C, 1, 1, 4, 0)
    first = dict(tiled=blob_a, bias=_dev(ba), O=Oa, kernel_size=(k, k), crop=(0, 0), bits=4 | U,
                 scale=_dev(scale_a), shift=_dev(shift_a), relu=True, emit=((1, 1), 16, 16, torch.int32),
                 want_float=False)
    second = dict(tiled=blob_b, bias=_dev(bb), O=Ob, kernel_size=(1, 1), crop=(p, p), bits=4 | U,
                  scale=_dev(scale_b), shift=_dev(shift_b), residual=_dev(res_b), relu=False, want_float=True)
    (oa, qa), (ob, qb) = kernels.conv2d_tiled_fused_pair(_dev(xp), (st, st), 16, first, second)
    va = so.np_dequantize_affine(ya, 16, scale_a, shift_a, None, True)
    vb = so.np_dequantize_affine(yb, 16, scale_b, shift_b, res_b, False)
    assert oa is None and qb is None
    np.testing.assert_array_equal(qa.cpu().numpy(), so.np_requantize(va, 16, 16, (1, 1)))
    np.testing.assert_array_equal(ob.cpu().numpy(), vb)
    # the other way round: float from the first, fixed point (int8 format) from the shortcut
    first.update(want_float=True, emit=None)
    second.update(want_float=False, emit=((0, 0), 3, 5, torch.int8), residual=None)
    (oa, qa), (ob, qb) = kernels.conv2d_tiled_fused_pair(_dev(xp), (st, st), 16, first, second)
    np.testing.assert_array_equal(oa.cpu().numpy(), va)
    vb2 = so.np_dequantize_affine(yb, 16, scale_b, shift_b, None, False)
    np.testing.assert_array_equal(qb.cpu().numpy().astype(np.int32), so.np_requantize(vb2, 3, 5, (0, 0)))
    # what cannot share a launch is refused
    bad = dict(second, bits=3)
    with pytest.raises(ValueError):
        kernels.conv2d_tiled_fused_pair(_dev(xp), (st, st), 16, first, bad)
    with pytest.raises(ValueError):
        kernels.conv2d_tiled_fused_pair(_dev(xp), (st, st), 16, first, dict(second, crop=(0, 0)))


def test_fused_resnet18_pairs_its_shortcuts():
    """fuse_conv_epilogues on a ResNet-18: the three down-sampling blocks run their first convolution and
    their shortcut as one launch, and the network output equals the pipeline without the in-kernel
    epilogue (int32 sums + separate conversion passes, separate shortcut launches) bit for bit."""
    from deepshift_amd import convert, fuse, modules, workloads
    g = torch.Generator().manual_seed(7)
    model = workloads.randomize_batchnorm(workloads.ResNet18(), g).eval()
    model, _ = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True)
    model = model.to(DEV)
    convert.round_shift_weights(model)
    x = torch.randn(4, 3, 96, 96, generator=g).to(DEV)
    with torch.no_grad():
        fused = fuse.fuse_conv_epilogues(model)
        pairs = [m for m in fused.modules() if isinstance(m, fuse.FusedShortcutPair)]
        assert len(pairs) == 3
        got = fused(x).clone()
        modules._FUSE_EPILOGUE = False
        try:
            plain = fuse.fuse_conv_epilogues(model, handoff=False)
            want = plain(x)
        finally:
            modules._FUSE_EPILOGUE = True
    assert torch.equal(got, want)


def test_fusable_covers_the_layers_of_a_small_image_network():
    """ds_conv2d_tiled_fusable at ResNet-20's shapes (batch 256): every convolution, the first one and the
    stride-2 ones included, has a fused launch; single images do not fill the machine and have none."""
    shapes = [(3, 34, 16, 1), (16, 34, 16, 1), (16, 34, 32, 2), (32, 18, 32, 1), (32, 18, 64, 2), (64, 10, 64, 1)]
    for C, Hp, O, st in shapes:
        assert kernels.conv2d_fusable((256, C, Hp, Hp), O, (3, 3), (st, st), 4 | U), (C, Hp, O, st)
    assert not kernels.conv2d_fusable((1, 16, 34, 34), 16, (3, 3), (1, 1), 4 | U)


@pytest.mark.parametrize("geom", [(3, 16, 34, 34, 16, 3, 3, (1, 1)), (2, 24, 20, 19, 64, 3, 3, (2, 1)),
                                  (2, 7, 11, 13, 40, 3, 2, (1, 1))], ids=lambda g: "x".join(str(v) for v in g[:7]))
def test_fused_five_bit_fields(oracle, rng, geom):
    """Fields of 5 bits (weight_bits 6: shifts down to -31, five codes per word) have no shift-plane form:
    every layer, 64 channels wide or not, takes the cooperative two-instruction launch."""
    Nb, C, Hp, Wp, O, FH, FW, stride = geom
    OH, OW = (Hp - FH) // stride[0] + 1, (Wp - FW) // stride[1] + 1
    xp = rng.integers(-2 ** 30, 2 ** 30, size=(Nb, C, Hp, Wp)).astype(np.int32)
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=31)
    bias = rng.integers(-2 ** 16, 2 ** 16, size=O).astype(np.int32)
    y = oracle.conv2d(xp, -s, sign, bias, stride, nthreads=NTHREADS)
    blob = kernels.tile_weights(_dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), 5)).reshape(-1),
                                O, C, FH, FW, 5, 0)
    scale = ((rng.random(O) + 0.5) * 2.0 ** -10).astype(np.float32)
    shift = rng.standard_normal(O).astype(np.float32)
    res = (rng.standard_normal((Nb, O, OH, OW)) * 2).astype(np.float32)
    for r, emit in ((res, (1, 1, 16, 16, torch.int32)), (None, (0, 2, 3, 5, torch.int8))):
        v = so.np_dequantize_affine(y, 16, scale, shift, r, True)
        out, q = abi_conv_fused(xp, blob, bias, O, FH, FW, stride, 5, 16, scale, shift, r, True, True, emit)
        np.testing.assert_array_equal(out, v)
        np.testing.assert_array_equal(q, so.np_requantize(v, emit[2], emit[3], emit[:2]))

