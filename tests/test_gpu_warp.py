"""GPU parity of cvcudaWarpAffine / cvcudaWarpPerspective [VarShape] Submit.

Exact-equality rows: the reference's table on tiny RGBA8 images with small integer and quarter-step
matrices, all five borders, three interpolations, forward and inverse maps
(tests/cvcuda/system/TestOpWarpAffine.cpp:232-319). Random rotations/scales: <= 1 LSB against the
reference's golden (oracle variant 0) and bit-exact against the restatement of this build's device
arithmetic: oracle variant 1 for NEAREST and CUBIC; on 8-bit pixels LINEAR is the 15-bit fixed-point blend
and CUBIC the 14-bit one (oracle variant 2); the bilinear one equals the golden wherever the weights are
dyadic (every row of the reference's table); LINEAR on the other types evaluates the bilinear sum in the
golden's own association, so variant 0 IS the device arithmetic there. BASELINE configuration 4 at full size."""
import itertools

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
NEAREST, LINEAR, CUBIC = 0, 1, 2
INVERSE_MAP = 16


def device_variant(interp, dtype=np.uint8):
    if interp != NEAREST and np.dtype(dtype) == np.uint8:
        return 2
    return 0 if interp == LINEAR else 1


def dyadic(values, bits=7):
    return all(float(v * (1 << bits)).is_integer() for v in values)

SIZES = [(5, 4, 5, 4), (5, 4, 6, 8), (7, 8, 4, 5)]
MATS = [(1, 0, 0, 0, 1, 0), (1, 0, 1, 0, 1, 2), (1, 2, 1, 2, 1, 2), (2, 2, 1, 3, 1, 2), (1, 2, 0, 1, 1, 0),
        (2, 2, 0, 3, 1, 1), (1, 0, 0, 0, 1, 1), (1, 2, 0, 2, 1, 1), (2, 2, 0, 3, 1, 0), (0.5, 2, 1, 0.75, 1, 2)]


def to_inverse(orc, m, inverse_given):
    return np.asarray(m, np.float32) if inverse_given else orc.invert_affine(m)


@pytest.mark.parametrize("interp", [NEAREST, LINEAR, CUBIC])
@pytest.mark.parametrize("border", [0, 1, 2, 3, 4])
def test_reference_table_exact(cv, orc, gpu, interp, border):
    op = cv.WarpAffine(0)
    for (sw, sh, dw, dh), m, inv in itertools.product(SIZES, MATS, (True, False)):
        src = orc.fill_u8((4, sh, sw, 4), sw * 100 + dh + int(m[1]))
        tin = cv.Tensor.from_numpy(src, "NHWC")
        tout = cv.Tensor.alloc([4, dh, dw, 4], np.uint8, "NHWC")
        op(None, tin, tout, m, interp | (INVERSE_MAP if inv else 0), border, (1, 2, 3, 4))
        torch.cuda.synchronize()
        res = tout.numpy()
        minv = to_inverse(orc, m, inv)
        dev = orc.warp(src, (dh, dw), minv, interp, border, (1, 2, 3, 4), variant=device_variant(interp))
        np.testing.assert_array_equal(res, dev, err_msg=str((sw, sh, dw, dh, m, inv)))
        gold = orc.warp(src, (dh, dw), minv, interp, border, (1, 2, 3, 4), variant=0)
        # LINEAR weights that are multiples of 2^-7 per axis are exact in the fixed-point blend as in float32
        exact = interp != CUBIC and dyadic(minv)
        tol = 0 if exact else 1
        assert np.abs(res.astype(np.int16) - gold.astype(np.int16)).max() <= tol, (sw, sh, dw, dh, m, inv)



@pytest.mark.parametrize("c", [1, 3, 4])
def test_tiny_sources_at_the_border_forms_limits(cv, orc, gpu, c):
    # 8-bit samples next to the image's edge take straight-line forms that fetch a pixel with one 4-byte load, moved
    # back where it would pass the image's last byte; images of under 4 bytes keep the generic loop. Sources of 1 to
    # 5 pixels (the mirroring and repeating borders' single folds do not reach that far: generic loop), every
    # interpolation and border mode: exact against the restatement.
    op = cv.WarpAffine(0)
    m = [0.8, 0.3, -0.4, -0.2, 0.9, 0.6]
    for (sw, sh) in [(1, 1), (2, 1), (1, 2), (3, 1), (1, 4), (2, 2), (5, 1), (1, 5)]:
        src = orc.fill_u8((2, sh, sw, c), 40 + sw * 7 + sh)
        for interp, border in itertools.product((NEAREST, LINEAR, CUBIC), (0, 1, 2, 3, 4)):
            tout = cv.Tensor.alloc([2, 6, 9, c], np.uint8, "NHWC")
            op(None, cv.Tensor.from_numpy(src, "NHWC"), tout, m, interp | INVERSE_MAP, border, (9, 200, 31, 77))
            torch.cuda.synchronize()
            dev = orc.warp(src, (6, 9), np.asarray(m, np.float32), interp, border, (9, 200, 31, 77), variant=device_variant(interp))
            np.testing.assert_array_equal(tout.numpy(), dev, err_msg=str((sw, sh, c, interp, border)))



@pytest.mark.parametrize("c", [1, 3, 4])
def test_mirroring_and_repeating_borders_near_and_far(cv, orc, gpu, c):
    # Under REFLECT, WRAP and REFLECT101 samples whose taps lie within one image size of the image take straight-line
    # forms with a single fold of the index; farther out the generic loop with its modulo. A destination 5 times the
    # source's size around it, shifted and slightly rotated, has both kinds in every interpolation: exact.
    op = cv.WarpAffine(0)
    sw, sh = 23, 17
    src = orc.fill_u8((2, sh, sw, c), 77 + c)
    m = [0.93, 0.11, -2.3 * sw, -0.07, 1.04, -1.9 * sh]  # destination (0, 0) maps about two image sizes in front
    for interp, border in itertools.product((NEAREST, LINEAR, CUBIC), (2, 3, 4)):
        tout = cv.Tensor.alloc([2, 5 * sh, 5 * sw, c], np.uint8, "NHWC")
        op(None, cv.Tensor.from_numpy(src, "NHWC"), tout, m, interp | INVERSE_MAP, border, (0, 0, 0, 0))
        torch.cuda.synchronize()
        dev = orc.warp(src, (5 * sh, 5 * sw), np.asarray(m, np.float32), interp, border, (0, 0, 0, 0), variant=device_variant(interp))
        np.testing.assert_array_equal(tout.numpy(), dev, err_msg=str((c, interp, border)))


def rotation(w, h, deg, s):
    t = np.deg2rad(deg)
    c, sn = s * np.cos(t), s * np.sin(t)
    cx, cy = (w - 1) / 2.0, (h - 1) / 2.0
    return [c, -sn, cx - c * cx + sn * cy, sn, c, cy - sn * cx - c * cy]


@pytest.mark.parametrize("dt,c", [(np.uint8, 3), (np.uint8, 1), (np.uint8, 4), (np.uint16, 3), (np.int16, 4),
                                  (np.float32, 1), (np.float32, 3)])
@pytest.mark.parametrize("interp", [NEAREST, LINEAR, CUBIC])
def test_random_rotations_tensor(cv, orc, gpu, dt, c, interp):
    n, h, w = 2, 97, 131
    if dt == np.float32:
        src = orc.fill_f32((n, h, w, c), 7) * 255
    else:
        src = orc.fill_u8((n, h, w, c, np.dtype(dt).itemsize), 7).view(dt).reshape(n, h, w, c)
    op = cv.WarpAffine(0)
    for deg, s, border in [(17.0, 1.1, 0), (-29.0, 0.85, 1), (5.5, 1.0, 4), (30.0, 1.2, 3), (-11.0, 0.9, 2)]:
        m = rotation(w, h, deg, s)
        tout = cv.Tensor.alloc([n, 80, 150, c], dt, "NHWC")
        op(None, cv.Tensor.from_numpy(src, "NHWC"), tout, m, interp, border, (9, 8, 7, 6))
        torch.cuda.synchronize()
        res = tout.numpy()
        minv = orc.invert_affine(m)
        dev = orc.warp(src, (80, 150), minv, interp, border, (9, 8, 7, 6), variant=device_variant(interp, dt))
        if dt == np.float32:
            assert np.abs(res - dev).max() <= 1e-3
        else:
            np.testing.assert_array_equal(res, dev)
            if dt == np.uint8 and interp != NEAREST:
                gold = orc.warp(src, (80, 150), minv, interp, border, (9, 8, 7, 6), variant=0)
                assert np.abs(res.astype(np.int16) - gold.astype(np.int16)).max() <= 1


def make_c4_batch(cv, K, orc, n, seed):
    rng = np.random.default_rng(seed)
    bi, bo, hosts, outs, mats = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], [], []
    for i in range(n):
        w, h = int(rng.integers(640, 1921)), int(rng.integers(480, 1081))
        a = orc.fill_u8((h, w, 3), 0xC0FFEE04 + i)
        hosts.append(a)
        bi.push_back(cv.Image.from_numpy(a, K.IMAGE_FORMAT_RGB8))
        o = cv.Image.alloc((w, h), K.IMAGE_FORMAT_RGB8)
        outs.append(o)
        bo.push_back(o)
        mats.append(rotation(w, h, float(rng.uniform(-30, 30)), float(rng.uniform(0.8, 1.2))))
    return bi, bo, hosts, outs, np.asarray(mats, np.float32)


def test_config4_varshape_full_size(cv, K, orc, gpu):
    # BASELINE config 4: 32 u8 RGB images, sizes in [640,1920]x[480,1080], rotation +-30deg / scale
    # 0.8-1.2 about the centre as forward maps, bilinear, constant border 0; <= 1 LSB vs golden
    n = 32
    bi, bo, hosts, outs, mats = make_c4_batch(cv, K, orc, n, 4)
    txf = cv.Tensor.from_numpy(mats, "NW")
    cv.WarpAffine(n)(None, bi, bo, txf, LINEAR, 0, (0, 0, 0, 0))
    torch.cuda.synchronize()
    for i in range(n):
        a, o = hosts[i], outs[i]
        res = o.plane_view(0, np.uint8, 3).cpu().numpy()
        minv = orc.invert_affine(mats[i])
        gold = orc.warp(a[None], a.shape[:2], minv, LINEAR, 0, (0, 0, 0, 0), variant=0, threads=1)[0]
        assert np.abs(res.astype(np.int16) - gold.astype(np.int16)).max() <= 1
        assert (res != gold).mean() < 0.02  # the fixed-point blend rounds differently on about 1 % of the bytes
        if i < 4:
            dev = orc.warp(a[None], a.shape[:2], minv, LINEAR, 0, (0, 0, 0, 0), variant=2)[0]
            np.testing.assert_array_equal(res, dev)


def test_varshape_small_all_modes_and_inverse_flag(cv, K, orc, gpu):
    rng = np.random.default_rng(11)
    n = 5
    bi, bo, hosts, outs, mats = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], [], []
    for i in range(n):
        w, h = int(rng.integers(20, 120)), int(rng.integers(20, 90))
        dw, dh = int(rng.integers(20, 140)), int(rng.integers(20, 100))
        a = orc.fill_u8((h, w, 4), 200 + i)
        hosts.append(a)
        bi.push_back(cv.Image.from_numpy(a, K.IMAGE_FORMAT_RGBA8))
        o = cv.Image.alloc((dw, dh), K.IMAGE_FORMAT_RGBA8)
        outs.append(o)
        bo.push_back(o)
        mats.append(rotation(w, h, float(rng.uniform(-40, 40)), float(rng.uniform(0.7, 1.4))))
    mats = np.asarray(mats, np.float32)
    op = cv.WarpAffine(8)
    for interp, border, inv in itertools.product((NEAREST, LINEAR, CUBIC), range(5), (False, True)):
        op(None, bi, bo, cv.Tensor.from_numpy(mats, "NW"), interp | (INVERSE_MAP if inv else 0), border,
           (10, 20, 30, 40))
        torch.cuda.synchronize()
        for i in range(n):
            w, h = outs[i].size
            res = outs[i].plane_view(0, np.uint8, 4).cpu().numpy()
            minv = mats[i] if inv else orc.invert_affine(mats[i])
            dev = orc.warp(hosts[i][None], (h, w), minv, interp, border, (10, 20, 30, 40), variant=device_variant(interp))[0]
            np.testing.assert_array_equal(res, dev, err_msg=str((interp, border, inv, i)))
    with pytest.raises(cv.Error) as e:
        cv.WarpAffine(4)(None, bi, bo, cv.Tensor.from_numpy(mats, "NW"), LINEAR)  # batch 5 > max 4
    assert e.value.status == 2
    with pytest.raises(cv.Error) as e:
        cv.WarpAffine(0)(None, bi, bo, cv.Tensor.from_numpy(mats, "NW"), LINEAR)
    assert e.value.status == 2


def homography_inverse(m):
    f = np.asarray(m, np.float32)
    d = f[0] * (f[4] * f[8] - f[5] * f[7]) + f[1] * (f[5] * f[6] - f[3] * f[8]) + f[2] * (f[3] * f[7] - f[4] * f[6])
    return np.array([(f[4] * f[8] - f[5] * f[7]) / d, -(f[1] * f[8] - f[2] * f[7]) / d, (f[1] * f[5] - f[2] * f[4]) / d,
                     -(f[3] * f[8] - f[5] * f[6]) / d, (f[0] * f[8] - f[2] * f[6]) / d, -(f[0] * f[5] - f[2] * f[3]) / d,
                     (f[3] * f[7] - f[4] * f[6]) / d, -(f[0] * f[7] - f[1] * f[6]) / d, (f[0] * f[4] - f[1] * f[3]) / d],
                    np.float32)


def test_warp_perspective(cv, K, orc, gpu):
    src = orc.fill_u8((2, 60, 80, 3), 21)
    H = [1.05, 0.08, -3.0, -0.04, 0.97, 2.0, 2e-4, -1e-4, 1.0]
    op = cv.WarpPerspective(4)
    for interp, border in itertools.product((NEAREST, LINEAR, CUBIC), (0, 1, 4)):
        for inv in (True, False):
            tout = cv.Tensor.alloc([2, 50, 90, 3], np.uint8, "NHWC")
            op(None, cv.Tensor.from_numpy(src, "NHWC"), tout, H, interp | (INVERSE_MAP if inv else 0), border,
               (5, 6, 7, 0))
            torch.cuda.synchronize()
            minv = np.asarray(H, np.float32) if inv else homography_inverse(H)
            ref = orc.warp(src, (50, 90), minv, interp, border, (5, 6, 7, 0), perspective=True, variant=device_variant(interp))
            d = np.abs(tout.numpy().astype(np.int16) - ref.astype(np.int16))
            # 1/x on the device is correctly rounded like the host's; allow 1 LSB for the inverse path whose
            # matrix entries come from float divisions evaluated on host in this test
            assert d.max() <= (0 if inv else 1)
    # var-shape: two images, matrices in a [N,9] tensor
    bi, bo = cv.ImageBatchVarShape(2), cv.ImageBatchVarShape(2)
    outs = []
    for i in range(2):
        bi.push_back(cv.Image.from_numpy(src[i], K.IMAGE_FORMAT_RGB8))
        o = cv.Image.alloc((90, 50), K.IMAGE_FORMAT_RGB8)
        outs.append(o)
        bo.push_back(o)
    mats = np.asarray([H, H], np.float32)
    op(None, bi, bo, cv.Tensor.from_numpy(mats, "NW"), LINEAR | INVERSE_MAP, 1, (0, 0, 0, 0))
    torch.cuda.synchronize()
    ref = orc.warp(src, (50, 90), H, LINEAR, 1, perspective=True, variant=2)
    for i in range(2):
        np.testing.assert_array_equal(outs[i].plane_view(0, np.uint8, 3).cpu().numpy(), ref[i])


# seeded random cases: every element type and channel count, interpolation and border mode; sources and outputs from 1
# pixel to 1400 x 900; rotations by any angle with independent axis scales of 0.4 to 2.5 and a shear, mapped near the
# source's centre or far outside it; affine and perspective; tensors and image batches of mixed sizes. Inverse maps
# are given, so device and oracle start from the same float32 matrix: exact for integers, 1e-3 for float32.
@pytest.mark.parametrize("seed", [31, 32])
def test_random_cases(cv, K, orc, gpu, seed):
    rng = np.random.default_rng(seed)
    fmts = {(np.uint8, 1): "U8", (np.uint8, 3): "RGB8", (np.uint8, 4): "RGBA8", (np.float32, 1): "F32", (np.float32, 3): "RGBf32"}
    types = [(np.uint8, 3), (np.uint8, 3), (np.uint8, 1), (np.uint8, 4), (np.uint16, 3), (np.int16, 1), (np.float32, 3),
             (np.float32, 4), (np.float32, 1)]
    for it in range(150):
        dt, c = types[int(rng.integers(0, len(types)))]
        interp, border, n = int(rng.integers(0, 3)), int(rng.integers(0, 5)), int(rng.integers(1, 4))
        persp = rng.random() < 0.3
        varshape = (dt, c) in fmts and rng.random() < 0.5
        big = rng.random() < 0.2
        bval = tuple(float(v) for v in rng.integers(0, 255, 4))

        def size():
            if big:
                return int(rng.integers(300, 1400)), int(rng.integers(200, 900))
            return int(rng.integers(1, 200)), int(rng.integers(1, 150))

        def matrix(sw, sh, dw, dh):
            t = np.deg2rad(float(rng.uniform(-180, 180)) if rng.random() < 0.8 else float(rng.choice([0, 90, 180, 45])))
            sx, sy = float(np.exp(rng.uniform(-0.9, 0.9))), float(np.exp(rng.uniform(-0.9, 0.9)))
            a, b, d, e = sx * np.cos(t), -sy * np.sin(t) + float(rng.uniform(-0.2, 0.2)), sx * np.sin(t), sy * np.cos(t)
            off = float(rng.uniform(-0.3, 0.3)) if rng.random() < 0.85 else float(rng.uniform(-3, 3))
            cx, cy = (sw - 1) / 2 + off * sw, (sh - 1) / 2 + off * sh
            m = [a, b, cx - a * (dw - 1) / 2 - b * (dh - 1) / 2, d, e, cy - d * (dw - 1) / 2 - e * (dh - 1) / 2]
            if persp:
                m += [float(rng.uniform(-2e-4, 2e-4)), float(rng.uniform(-2e-4, 2e-4)), 1.0]
            return np.asarray(m, np.float32)

        def image(h, w, s):
            if dt == np.float32:
                return orc.fill_f32((h, w, c), s) * 255
            return orc.fill_u8((h, w, c, np.dtype(dt).itemsize), s).view(dt).reshape(h, w, c)

        def compare(res, src, hw, m, what):
            dev = orc.warp(src, hw, m, interp, border, bval, perspective=persp, variant=device_variant(interp, dt))
            case = "seed %d case %d %s: %s x%d interp %d border %d persp %d %s -> %s m %s" % (
                seed, it, what, np.dtype(dt).name, c, interp, border, persp, src.shape, hw, m.tolist())
            if dt == np.float32:
                assert np.abs(res - dev).max() <= 1e-3, case
            else:
                np.testing.assert_array_equal(res, dev, err_msg=case)

        op = (cv.WarpPerspective if persp else cv.WarpAffine)(8)
        if varshape:
            fmt = getattr(K, "IMAGE_FORMAT_" + fmts[(dt, c)])
            bi, bo, hosts, outs, mats = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], [], []
            for i in range(n):
                (sw, sh), (dw, dh) = size(), size()
                hosts.append(image(sh, sw, 100 * it + i + seed))
                bi.push_back(cv.Image.from_numpy(hosts[-1], fmt))
                outs.append(cv.Image.alloc((dw, dh), fmt))
                bo.push_back(outs[-1])
                mats.append(matrix(sw, sh, dw, dh))
            mats = np.asarray(mats, np.float32)
            op(None, bi, bo, cv.Tensor.from_numpy(mats, "NW"), interp | INVERSE_MAP, border, bval)
            torch.cuda.synchronize()
            for i in range(n):
                w, h = outs[i].size
                compare(outs[i].plane_view(0, dt, c).cpu().numpy()[None], hosts[i][None], (h, w), mats[i], "image %d" % i)
        else:
            (sw, sh), (dw, dh) = size(), size()
            src = np.stack([image(sh, sw, 100 * it + i + seed) for i in range(n)])
            m = matrix(sw, sh, dw, dh)
            tout = cv.Tensor.alloc([n, dh, dw, c], dt, "NHWC")
            op(None, cv.Tensor.from_numpy(src, "NHWC"), tout, m.tolist(), interp | INVERSE_MAP, border, bval)
            torch.cuda.synchronize()
            compare(tout.numpy(), src, (dh, dw), m, "tensor")


def test_tensor_negative(cv, gpu):
    op = cv.WarpAffine(0)
    a = cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC")
    ident = [1, 0, 0, 0, 1, 0]
    for out, flags, border in [(cv.Tensor.alloc([2, 8, 8, 3], np.float32, "NHWC"), LINEAR, 0),
                               (cv.Tensor.alloc([3, 8, 8, 3], np.uint8, "NHWC"), LINEAR, 0),
                               (cv.Tensor.alloc([2, 8, 8, 4], np.uint8, "NHWC"), LINEAR, 0),
                               (cv.Tensor.alloc([2, 3, 8, 8], np.uint8, "NCHW"), LINEAR, 0),
                               (cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC"), 3, 0),     # AREA
                               (cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC"), LINEAR, 9)]:
        with pytest.raises(cv.Error) as e:
            op(None, a, out, ident, flags, border)
        assert e.value.status == 2
