"""Size-independent properties of the operators at the BASELINE configurations' full sizes: round trips,
idempotence, identities, linearity and agreement between operators that must produce the same bytes. The inputs stay
on the device and results are compared there, so every case runs on whole batches that a CPU oracle would take
minutes for; the oracle-backed parity tests cover the same kernels at sizes it finishes in seconds."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

NEAREST, LINEAR, CUBIC, AREA = 0, 1, 2, 3


def device_u8(gpu, shape, seed):
    g = torch.Generator(device=gpu)
    g.manual_seed(seed)
    return torch.randint(0, 256, shape, dtype=torch.uint8, device=gpu, generator=g)


def tensor_from(cv, t, layout):
    out = cv.Tensor.alloc(list(t.shape), np.dtype(str(t.dtype).replace("torch.", "")), layout)
    out.torch_view().copy_(t)
    return out


def test_streaming_operators_round_trip_on_a_1080p_batch(cv, K, gpu):
    n, h, w = 32, 1080, 1920
    src = device_u8(gpu, (n, h, w, 3), 1)
    tin = tensor_from(cv, src, "NHWC")
    a = cv.Tensor.alloc([n, h, w, 3], np.uint8, "NHWC")
    b = cv.Tensor.alloc([n, h, w, 3], np.uint8, "NHWC")
    # channel reversal twice, alpha added then dropped
    cvt = cv.CvtColor()
    cvt(None, tin, a, K.COLOR_BGR2RGB)
    assert torch.equal(a.torch_view(), src.flip(-1))
    cvt(None, a, b, K.COLOR_RGB2BGR)
    assert torch.equal(b.torch_view(), src)
    rgba = cv.Tensor.alloc([n, h, w, 4], np.uint8, "NHWC")
    cvt(None, tin, rgba, K.COLOR_BGR2BGRA)
    assert torch.equal(rgba.torch_view()[..., :3], src) and bool((rgba.torch_view()[..., 3] == 255).all())
    cvt(None, rgba, b, K.COLOR_BGRA2BGR)
    assert torch.equal(b.torch_view(), src)
    # mirrors: each twice is the identity, both at once equals one after the other
    flip = cv.Flip()
    for code, dims in ((0, (1,)), (1, (2,)), (-1, (1, 2))):
        flip(None, tin, a, code)
        assert torch.equal(a.torch_view(), src.flip(dims))
        flip(None, a, b, code)
        assert torch.equal(b.torch_view(), src)
    # layout change and back
    planar = cv.Tensor.alloc([n, 3, h, w], np.uint8, "NCHW")
    cv.Reformat()(None, tin, planar)
    assert torch.equal(planar.torch_view(), src.permute(0, 3, 1, 2))
    cv.Reformat()(None, planar, b)
    assert torch.equal(b.torch_view(), src)
    # u8 -> f32 -> u8 with exact scales
    f = cv.Tensor.alloc([n, h, w, 3], np.float32, "NHWC")
    cv.ConvertTo()(None, tin, f, 0.5, 3.0)
    assert torch.equal(f.torch_view(), src.float() * 0.5 + 3.0)
    cv.ConvertTo()(None, f, b, 2.0, -6.0)
    assert torch.equal(b.torch_view(), src)
    # Normalize with base 0 and scale 1 copies; (x - b) * s in float32 is the elementwise expression
    zero = cv.Tensor.from_numpy(np.zeros((1, 1, 1, 3), np.float32), "NHWC")
    one = cv.Tensor.from_numpy(np.ones((1, 1, 1, 3), np.float32), "NHWC")
    cv.Normalize()(None, tin, zero, one, b)
    assert torch.equal(b.torch_view(), src)
    base = np.array([[[[10.0, 20.5, 128.0]]]], np.float32)
    scale = np.array([[[[0.5, 2.0, 0.25]]]], np.float32)
    cv.ConvertTo()(None, tin, f, 1.0, 0.0)
    g = cv.Tensor.alloc([n, h, w, 3], np.float32, "NHWC")
    cv.Normalize()(None, f, cv.Tensor.from_numpy(base, "NHWC"), cv.Tensor.from_numpy(scale, "NHWC"), g)
    want = (src.float() - torch.from_numpy(base).to(gpu)) * torch.from_numpy(scale).to(gpu)
    assert torch.equal(g.torch_view(), want)
    # crops of the whole image and centred crops
    cv.CustomCrop()(None, tin, b, (0, 0, w, h))
    assert torch.equal(b.torch_view(), src)
    c = cv.Tensor.alloc([n, 224, 224, 3], np.uint8, "NHWC")
    cv.CenterCrop()(None, tin, c, (224, 224))
    assert torch.equal(c.torch_view(), src[:, (h - 224) // 2:(h - 224) // 2 + 224, (w - 224) // 2:(w - 224) // 2 + 224])


def test_resize_and_warp_identities_on_a_1080p_batch(cv, K, gpu):
    n, h, w = 8, 1080, 1920
    src = device_u8(gpu, (n, h, w, 3), 2)
    tin = tensor_from(cv, src, "NHWC")
    out = cv.Tensor.alloc([n, h, w, 3], np.uint8, "NHWC")
    for interp in (NEAREST, LINEAR):
        out.torch_view().zero_()
        cv.Resize()(None, tin, out, interp)
        assert torch.equal(out.torch_view(), src), interp
    # an exact 2x reduction with NEAREST picks the odd rows and columns (floor((d + .5) * 2) = 2d + 1)
    half = cv.Tensor.alloc([n, h // 2, w // 2, 3], np.uint8, "NHWC")
    cv.Resize()(None, tin, half, NEAREST)
    assert torch.equal(half.torch_view(), src[:, 1::2, 1::2])
    # ... and bilinear averages each 2 x 2 block (weights .25 each; the sum of four bytes over 4 in float32 is exact,
    # ties go to the even integer)
    cv.Resize()(None, tin, half, LINEAR)
    blocks = src.float().reshape(n, h // 2, 2, w // 2, 2, 3)
    mean = (blocks[:, :, 0, :, 0] * 0.25 + blocks[:, :, 0, :, 1] * 0.25 + blocks[:, :, 1, :, 0] * 0.25
            + blocks[:, :, 1, :, 1] * 0.25)
    assert torch.equal(half.torch_view(), torch.round(mean).to(torch.uint8))
    # the box filter of an exact 2x reduction is the same block mean (weights 2^-1 per axis, nothing rounded before
    # the last step), and at equal sizes it is a copy
    cv.Resize()(None, tin, half, AREA)
    assert torch.equal(half.torch_view(), torch.round(mean).to(torch.uint8))
    out.torch_view().zero_()
    cv.Resize()(None, tin, out, AREA)
    assert torch.equal(out.torch_view(), src)
    # 1080p -> 720p (scale 1.5): output pixel (2i, 2j) covers source pixel (3i, 3j) and half of the next along each
    # axis, so with weights 4/9, 2/9, 2/9, 1/9 it is within rounding of that sum everywhere
    small = cv.Tensor.alloc([n, 720, 1280, 3], np.uint8, "NHWC")
    cv.Resize()(None, tin, small, AREA)
    f = src.double()
    want = (4 * f[:, 0::3, 0::3] + 2 * f[:, 0::3, 1::3] + 2 * f[:, 1::3, 0::3] + f[:, 1::3, 1::3]) / 9
    got = small.torch_view()[:, 0::2, 0::2].double()
    assert float((got - want).abs().max()) <= 0.5 + 1e-2
    # warps: the identity map, and a whole-pixel shift with a constant border
    warp = cv.WarpAffine(0)
    for interp in (NEAREST, LINEAR, CUBIC):
        out.torch_view().zero_()
        warp(None, tin, out, [1, 0, 0, 0, 1, 0], interp, 0, (0, 0, 0, 0))
        assert torch.equal(out.torch_view(), src), interp
    dx, dy = 37, 11
    warp(None, tin, out, [1, 0, dx, 0, 1, dy], LINEAR, 0, (9, 8, 7, 0))
    got = out.torch_view()
    assert torch.equal(got[:, dy:, dx:], src[:, :h - dy, :w - dx])
    border = torch.tensor([9, 8, 7], dtype=torch.uint8, device=gpu)
    assert bool((got[:, :dy] == border).all()) and bool((got[:, :, :dx] == border).all())
    # the projective operator with an affine matrix is the affine operator
    m = [0.9, -0.2, 30.0, 0.25, 1.1, -12.0]
    out2 = cv.Tensor.alloc([n, h, w, 3], np.uint8, "NHWC")
    warp(None, tin, out, m, LINEAR, 0, (0, 0, 0, 0))
    cv.WarpPerspective(0)(None, tin, out2, m + [0, 0, 1], LINEAR, 0, (0, 0, 0, 0))
    assert torch.equal(out.torch_view(), out2.torch_view())


def test_fused_operator_agrees_with_the_operators_it_fuses_at_full_size(cv, K, gpu):
    n, h, w = 64, 1080, 1920
    src = device_u8(gpu, (n, h, w, 3), 3)
    tin = tensor_from(cv, src, "NHWC")
    fused = cv.ResizeCropConvertReformat()
    # no resize (resizeDim = source size): a crop, a conversion and a layout change
    out = cv.Tensor.alloc([n, 3, 224, 224], np.float32, "NCHW")
    fused(None, tin, out, (w, h), LINEAR, (115, 16), 0, 0.5, 1.0, False)
    want = src[:, 16:16 + 224, 115:115 + 224].permute(0, 3, 1, 2).float() * 0.5 + 1.0
    assert torch.equal(out.torch_view(), want)
    # NEAREST at the benchmark geometry equals Resize NEAREST to 455 x 256 followed by the crop
    resized = cv.Tensor.alloc([n, 256, 455, 3], np.uint8, "NHWC")
    cv.Resize()(None, tin, resized, NEAREST)
    nn = cv.Tensor.alloc([n, 224, 224, 3], np.uint8, "NHWC")
    fused(None, tin, nn, (455, 256), NEAREST, (115, 16), 0, 1.0, 0.0, True)
    assert torch.equal(nn.torch_view(), resized.torch_view()[:, 16:16 + 224, 115:115 + 224])
    # channel reversal in the fused operator equals a reversal afterwards; interleaved and planar outputs hold the
    # same values
    a = cv.Tensor.alloc([n, 224, 224, 3], np.float32, "NHWC")
    b = cv.Tensor.alloc([n, 224, 224, 3], np.float32, "NHWC")
    fused(None, tin, a, (455, 256), LINEAR, (115, 16), 0, 1 / 255.0, 0.0, False)
    fused(None, tin, b, (455, 256), LINEAR, (115, 16), K.CHANNEL_REVERSE, 1 / 255.0, 0.0, False)
    assert torch.equal(b.torch_view(), a.torch_view().flip(-1))
    fused(None, tin, out, (455, 256), LINEAR, (115, 16), 0, 1 / 255.0, 0.0, False)
    assert torch.equal(out.torch_view(), a.torch_view().permute(0, 3, 1, 2))
    # the result does not depend on what else is in the batch: sample 63 alone equals sample 63 of the batch
    alone = cv.Tensor.alloc([1, 3, 224, 224], np.float32, "NCHW")
    fused(None, tensor_from(cv, src[63:64], "NHWC"), alone, (455, 256), LINEAR, (115, 16), 0, 1 / 255.0, 0.0, False)
    assert torch.equal(alone.torch_view()[0], out.torch_view()[63])


def test_colour_round_trips_on_a_1080p_batch(cv, K, gpu):
    n, h, w = 32, 1080, 1920
    # an image whose 2 x 2 blocks are one colour loses nothing to chroma subsampling: BGR -> NV12 -> BGR returns it
    # within the two roundings of the fixed-point formulas
    small = device_u8(gpu, (n, h // 2, w // 2, 3), 4)
    src = small.repeat_interleave(2, dim=1).repeat_interleave(2, dim=2).contiguous()
    tin = tensor_from(cv, src, "NHWC")
    nv12 = cv.Tensor.alloc([n, h * 3 // 2, w, 1], np.uint8, "NHWC")
    back = cv.Tensor.alloc([n, h, w, 3], np.uint8, "NHWC")
    cv.CvtColor()(None, tin, nv12, K.COLOR_BGR2YUV_NV12)
    cv.CvtColor()(None, nv12, back, K.COLOR_YUV2BGR_NV12)
    diff = (back.torch_view().int() - src.int()).abs()
    # colours outside the encoder's range are clipped (Y to [16, 235] and the like); the bulk must be close
    assert float((diff <= 3).float().mean()) > 0.97 and int(diff.max()) < 64
    # NV12 and NV21 differ by the order of the chroma pair only; the planar forms hold the same samples
    nv21 = cv.Tensor.alloc([n, h * 3 // 2, w, 1], np.uint8, "NHWC")
    cv.CvtColor()(None, tin, nv21, K.COLOR_BGR2YUV_NV21)
    a, b = nv12.torch_view(), nv21.torch_view()
    assert torch.equal(a[:, :h], b[:, :h])
    assert torch.equal(a[:, h:, 0::2], b[:, h:, 1::2]) and torch.equal(a[:, h:, 1::2], b[:, h:, 0::2])
    i420 = cv.Tensor.alloc([n, h * 3 // 2, w, 1], np.uint8, "NHWC")
    cv.CvtColor()(None, tin, i420, K.COLOR_BGR2YUV_I420)
    c = i420.torch_view()
    assert torch.equal(c[:, :h], a[:, :h])
    u_plane = c[:, h:h + h // 4].reshape(n, h // 2, w // 2)
    v_plane = c[:, h + h // 4:].reshape(n, h // 2, w // 2)
    assert torch.equal(u_plane, a[:, h:, 0::2, 0]) and torch.equal(v_plane, a[:, h:, 1::2, 0])
    # decoding to RGB is decoding to BGR reversed; the luma rows are the gray image
    rgb = cv.Tensor.alloc([n, h, w, 3], np.uint8, "NHWC")
    cv.CvtColor()(None, nv12, rgb, K.COLOR_YUV2RGB_NV12)
    assert torch.equal(rgb.torch_view(), back.torch_view().flip(-1))
    gray = cv.Tensor.alloc([n, h, w, 1], np.uint8, "NHWC")
    cv.CvtColor()(None, nv12, gray, K.COLOR_YUV2GRAY_NV12)
    assert torch.equal(gray.torch_view(), a[:, :h])
    # gray -> BGR -> gray is exact (the three weights sum to 1 << 15)
    bgr = cv.Tensor.alloc([n, h, w, 3], np.uint8, "NHWC")
    g2 = cv.Tensor.alloc([n, h, w, 1], np.uint8, "NHWC")
    cv.CvtColor()(None, gray, bgr, K.COLOR_GRAY2BGR)
    cv.CvtColor()(None, bgr, g2, K.COLOR_BGR2GRAY)
    assert torch.equal(g2.torch_view(), gray.torch_view())


def test_image_batch_forms_on_32_images_of_mixed_sizes(cv, K, gpu):
    # the sizes of BASELINE configuration 4: W in [640, 1920], H in [480, 1080]
    rng = np.random.default_rng(4)
    sizes = [(int(rng.integers(640, 1921)) & ~1, int(rng.integers(480, 1081)) & ~3) for _ in range(32)]
    srcs = [device_u8(gpu, (h, w, 3), 100 + i) for i, (w, h) in enumerate(sizes)]

    def batch_of(tensors, fmt=None):
        b, images = cv.ImageBatchVarShape(len(tensors)), []
        for t in tensors:
            img = cv.Image.alloc((t.shape[1], t.shape[0]), fmt or K.IMAGE_FORMAT_RGB8)
            img.plane_view(0, np.uint8, t.shape[2]).copy_(t)
            images.append(img)
            b.push_back(img)
        return b, images

    def empty_like(shapes, fmt=None, c=3):
        return batch_of([torch.zeros((h, w, c), dtype=torch.uint8, device=gpu) for (w, h) in shapes], fmt)

    bin_, _ = batch_of(srcs)

    def views(images, c=3):
        return [i.plane_view(0, np.uint8, c) for i in images]

    # Resize to the same size and the identity warp return the images; a mirror twice as well
    for op, args in ((cv.Resize(), (NEAREST,)), (cv.Resize(), (LINEAR,))):
        bout, outs = empty_like(sizes)
        op(None, bin_, bout, *args)
        assert all(torch.equal(v, s) for v, s in zip(views(outs), srcs))
    ident = cv.Tensor.from_numpy(np.tile(np.array([1, 0, 0, 0, 1, 0], np.float32), (32, 1)), "NW")
    bout, outs = empty_like(sizes)
    cv.WarpAffine(32)(None, bin_, bout, ident, LINEAR, 0, (0, 0, 0, 0))
    assert all(torch.equal(v, s) for v, s in zip(views(outs), srcs))
    codes = cv.Tensor.from_numpy(np.full((32,), -1, np.int32), "N")
    bmid, mids = empty_like(sizes)
    cv.Flip()(None, bin_, bmid, codes)
    assert all(torch.equal(v, s.flip((0, 1))) for v, s in zip(views(mids), srcs))
    bout, outs = empty_like(sizes)
    cv.Flip()(None, bmid, bout, codes)
    assert all(torch.equal(v, s) for v, s in zip(views(outs), srcs))
    # colour: reversal twice; NV12 and back on images of constant 2 x 2 blocks
    bout, outs = empty_like(sizes)
    cv.CvtColor()(None, bin_, bmid, K.COLOR_BGR2RGB)
    cv.CvtColor()(None, bmid, bout, K.COLOR_RGB2BGR)
    assert all(torch.equal(v, s) for v, s in zip(views(outs), srcs))
    blocky = [s[::2, ::2].repeat_interleave(2, dim=0).repeat_interleave(2, dim=1).contiguous() for s in srcs]
    bblock, _ = batch_of(blocky)
    bnv, nvs = empty_like([(w, h * 3 // 2) for (w, h) in sizes], K.IMAGE_FORMAT_U8, 1)
    cv.CvtColor()(None, bblock, bnv, K.COLOR_BGR2YUV_NV12)
    bout, outs = empty_like(sizes)
    cv.CvtColor()(None, bnv, bout, K.COLOR_YUV2BGR_NV12)
    for v, s in zip(views(outs), blocky):
        diff = (v.int() - s.int()).abs()
        assert float((diff <= 3).float().mean()) > 0.97 and int(diff.max()) < 64
    # each image of the batch gives what the same image gives alone as a tensor
    t = cv.Tensor.alloc([1, sizes[31][1] * 3 // 2, sizes[31][0], 1], np.uint8, "NHWC")
    cv.CvtColor()(None, tensor_from(cv, blocky[31][None], "NHWC"), t, K.COLOR_BGR2YUV_NV12)
    assert torch.equal(t.torch_view()[0], views(nvs, 1)[31])
