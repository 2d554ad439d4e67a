"""GPU parity of cvcudaCropFlipNormalizeReformatSubmit against the oracle's restatement of the
reference golden, on the reference's parameter rows (tests/cvcuda/system/
TestOpCropFlipNormalizeReformat.cpp:411-447: sizes, formats, borders, base/scale shapes, flags) with
its input recipe (image sizes 0.8..1.1 x nominal, crop x/y from -3, flip codes -1..2, border value 1).
Tolerance 1e-4 as there (:407); integer outputs must match exactly."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
STDDEV = 1

# width, height, images, scalarBase, scalarScale, flags, gscale, shift, eps, src fmt, dst fmt, border, src type, dst type
ROWS = [
    (9, 13, 10, True, True, 0, 1.0, 0.0, 0.0, "RGB8p", "RGB8p", 0, np.uint8, np.uint8),
    (9, 13, 10, True, True, 0, 1.0, 0.0, 0.0, "RGB8p", "RGB8", 0, np.uint8, np.uint8),
    (9, 13, 10, True, True, 0, 1.0, 0.0, 0.0, "RGB8", "RGB8p", 0, np.uint8, np.uint8),
    (9, 13, 10, True, True, 0, 1.0, 0.0, 0.0, "RGBA8", "RGBA8", 0, np.uint8, np.uint8),
    (9, 13, 10, True, True, 0, 1.0, 0.0, 0.0, "RGBA8p", "RGBA8", 0, np.uint8, np.uint8),
    (9, 13, 10, True, True, 0, 1.0, 0.0, 0.0, "RGBA8", "RGBA8", 2, np.uint8, np.uint8),
    (9, 13, 10, True, True, 0, 1.0, 0.0, 0.0, "RGBA8", "RGBA8", 4, np.uint8, np.uint8),
    (10, 10, 2, True, True, 0, 1.0, 0.0, 0.0, "RGB8", "RGB8", 3, np.uint8, np.uint8),
    (15, 15, 3, True, True, 0, 1.0, 0.0, 0.0, "U8", "U8", 1, np.uint8, np.uint8),
    (9, 13, 10, True, True, 0, 1.0, 0.0, 0.0, "RGBA8p", "RGBAf32", 0, np.uint8, np.float32),
    (15, 15, 10, True, True, 0, 1.0, 0.0, 0.0, "F32", "F32", 1, np.float32, np.float32),
    (15, 15, 2, True, True, 0, 1.0, 0.0, 0.0, "S32", "F32", 1, np.int32, np.float32),
    (15, 15, 2, True, True, 0, 1.0, 0.0, 0.0, "S32", "S32", 1, np.int32, np.int32),
    (51, 53, 10, True, False, 0, 1.234, 33.21, 0.0, "RGBf32", "RGBf32", 1, np.float32, np.float32),
    (51, 53, 10, True, True, STDDEV, 1.1, 0.3, 1.23, "RGBAf32", "RGBAf32p", 1, np.float32, np.float32),
    (51, 53, 10, False, False, 0, 1.0, 12.3, 0.0, "RGBAf32p", "RGBAf32", 1, np.float32, np.float32),
    (51, 53, 10, False, True, STDDEV, 1.1, 0.3, 1.23, "RGBAf32", "RGBAf32p", 1, np.float32, np.float32),
    # beyond the reference's table: the classification pipeline shape (u8 RGB -> f32 NCHW, mean/std)
    (320, 240, 6, False, False, STDDEV, 1.0, 0.0, 0.0, "RGB8", "RGBf32p", 0, np.uint8, np.float32),
    (64, 48, 4, False, False, 0, 0.5, 3.0, 0.0, "RGB8", "RGB8", 2, np.uint8, np.int8),
    # 32-bit unsigned on either side (reference type tables OpCropFlipNormalizeReformat.cu:335-341, 449-454);
    # the inputs span the whole range, so results saturate at both ends
    (33, 21, 3, True, True, 0, 1.0, 0.0, 0.0, "U32", "U32", 0, np.uint32, np.uint32),
    (33, 21, 3, True, True, 0, 1.5, -7.0e8, 0.0, "U32", "U32", 1, np.uint32, np.uint32),
    (33, 21, 3, True, True, 0, 2.0e7, 0.0, 0.0, "U8", "U32", 0, np.uint8, np.uint32),
    (33, 21, 3, True, True, 0, 1.0, 0.0, 0.0, "U32", "F32", 2, np.uint32, np.float32),
]
CHANNELS = {"RGB8": 3, "RGB8p": 3, "RGBA8": 4, "RGBA8p": 4, "U8": 1, "F32": 1, "S32": 1, "U32": 1, "RGBf32": 3, "RGBf32p": 3,
            "RGBAf32": 4, "RGBAf32p": 4}


def make_image(cv, K, a, fmt_name):
    """a: [H,W,C] host array -> device image of the named format (planar formats: one plane per channel)."""
    fmt = getattr(K, "IMAGE_FORMAT_" + fmt_name)
    if not fmt_name.endswith("p"):
        return cv.Image.from_numpy(a, fmt)
    img = cv.Image.alloc((a.shape[1], a.shape[0]), fmt)
    for c in range(a.shape[2]):
        img.plane_view(c, a.dtype, 1).copy_(torch.from_numpy(np.ascontiguousarray(a[:, :, c:c + 1])).cuda())
    return img


@pytest.mark.parametrize("row", ROWS, ids=lambda r: "%dx%dx%d-%s-%s-b%d" % (r[0], r[1], r[2], r[9], r[10], r[11]))
def test_reference_rows(cv, K, orc, gpu, row):
    w, h, n, sbase, sscale, flags, gscale, shift, eps, sfmt, dfmt, border, ts, td = row
    c = CHANNELS[sfmt]
    rng = np.random.default_rng(w * 131 + h + n + border)
    batch, hosts = cv.ImageBatchVarShape(n), []
    for i in range(n):
        iw = int(rng.integers(int(w * 0.8), int(w * 1.1) + 1))
        ih = int(rng.integers(int(h * 0.8), int(h * 1.1) + 1))
        a = orc.fill_u8((ih, iw, c), 900 + i).astype(ts)
        if ts == np.uint32:
            a = a * np.uint32(0x01010101)
        if ts == np.float32:
            a = a + orc.fill_f32((ih, iw, c), 950 + i)
        hosts.append(a)
        batch.push_back(make_image(cv, K, a, sfmt))
    ow, oh = max(a.shape[1] for a in hosts), max(a.shape[0] for a in hosts)
    flips = rng.integers(-1, 3, n).astype(np.int32)
    crops = np.zeros((n, 1, 1, 4), np.int32)
    for i, a in enumerate(hosts):
        ih, iw = a.shape[:2]
        crops[i, 0, 0] = (rng.integers(-3, min(10, iw // 10) + 2), rng.integers(-3, min(10, ih // 10) + 2),
                          rng.integers(max(int(iw * 0.8), iw - 10), iw), rng.integers(max(int(ih * 0.8), ih - 10), ih))
    base = (orc.fill_f32((1, 1, 1, 1 if sbase else 4), 5) * 255).astype(np.float32)
    scale = orc.fill_f32((1, 1, 1, 1 if sscale else 4), 6)
    planar_out = dfmt.endswith("p")
    out = cv.Tensor.alloc([n, c, oh, ow] if planar_out else [n, oh, ow, c], td, "NCHW" if planar_out else "NHWC")
    if td != np.uint32:  # torch has no fill for 32-bit unsigned tensors; every element is written anyway
        out.torch_view().fill_(77)
    cv.CropFlipNormalizeReformat()(None, batch, out, cv.Tensor.from_numpy(crops, "NHWC"), border, 1.0,
                                   cv.Tensor.from_numpy(flips, "N"), cv.Tensor.from_numpy(base, "NHWC"),
                                   cv.Tensor.from_numpy(scale, "NHWC"), gscale, shift, eps, flags)
    torch.cuda.synchronize()
    got = out.numpy()
    if planar_out:
        got = got.transpose(0, 2, 3, 1)
    for i, a in enumerate(hosts):
        ref = orc.crop_flip_normalize(a, (oh, ow), td, crops[i, 0, 0], flips[i], border, 1.0,
                                      base.reshape(-1)[:c] if not sbase else base.reshape(-1),
                                      scale.reshape(-1)[:c] if not sscale else scale.reshape(-1), gscale, shift, eps,
                                      flags != 0)
        if np.dtype(td).kind == "f":
            assert np.abs(got[i] - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
        else:
            np.testing.assert_array_equal(got[i], ref)


def test_closed_forms_and_negative(cv, K, orc, gpu):
    # identity parameters: a plain crop, flipped; zero fill beyond the rectangle
    a = orc.fill_u8((40, 60, 3), 4)
    batch = cv.ImageBatchVarShape(1)
    batch.push_back(cv.Image.from_numpy(a, K.IMAGE_FORMAT_RGB8))
    out = cv.Tensor.alloc([1, 32, 48, 3], np.uint8, "NHWC")
    one, zero = np.ones((1, 1, 1, 1), np.float32), np.zeros((1, 1, 1, 1), np.float32)
    op = cv.CropFlipNormalizeReformat()
    for code, pick in [(2, lambda w: w), (1, lambda w: w[:, ::-1]), (0, lambda w: w[::-1]), (-1, lambda w: w[::-1, ::-1])]:
        crop = np.array([[[[5, 3, 40, 30]]]], np.int32)
        op(None, batch, out, cv.Tensor.from_numpy(crop, "NHWC"), 0, 0.0, cv.Tensor.from_numpy(np.array([code], np.int32), "N"),
           cv.Tensor.from_numpy(zero, "NHWC"), cv.Tensor.from_numpy(one, "NHWC"))
        torch.cuda.synchronize()
        res = out.numpy()[0]
        np.testing.assert_array_equal(res[:30, :40], pick(a[3:33, 5:45]))
        assert (res[30:] == 0).all() and (res[:, 40:] == 0).all()
    crop_t = cv.Tensor.from_numpy(np.array([[[[0, 0, 8, 8]]]], np.int32), "NHWC")
    flip_t = cv.Tensor.from_numpy(np.array([0], np.int32), "N")
    z, o = cv.Tensor.from_numpy(zero, "NHWC"), cv.Tensor.from_numpy(one, "NHWC")
    bad_calls = [
        (cv.Tensor.alloc([2, 32, 48, 3], np.uint8, "NHWC"), crop_t, 0, flip_t, z, o),          # batch size
        (cv.Tensor.alloc([1, 32, 48, 4], np.uint8, "NHWC"), crop_t, 0, flip_t, z, o),          # channels
        (cv.Tensor.alloc([32, 48, 3], np.uint8, "HWC"), crop_t, 0, flip_t, z, o),              # rank
        (out, cv.Tensor.from_numpy(np.zeros((1, 1, 1, 3), np.int32), "NHWC"), 0, flip_t, z, o),   # crop shape
        (out, crop_t, 9, flip_t, z, o),                                                        # border mode
        (out, crop_t, 0, cv.Tensor.from_numpy(np.zeros(1, np.float32), "N"), z, o),            # flip type
        (out, crop_t, 0, flip_t, cv.Tensor.from_numpy(np.zeros((1, 1, 1, 2), np.float32), "NHWC"), o),   # base channels
        (cv.Tensor.alloc([1, 32, 48, 3], np.float64, "NHWC"), crop_t, 0, flip_t, z, o),        # output type
    ]
    for t_out, t_crop, border, t_flip, t_base, t_scale in bad_calls:
        with pytest.raises(cv.Error) as e:
            op(None, batch, t_out, t_crop, border, 0.0, t_flip, t_base, t_scale)
        assert e.value.status == 2
