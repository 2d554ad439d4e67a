"""The reference's Python tests of the path's operators (tests/cvcuda/python/test_op{resize,cvtcolor,normalize,
reformat,convertto,customcrop,centercrop,flip,warpaffine,warpperspective,resizecropconvertreformat,
cropflipnormalizereformat}.py), restated against cvcuda_amd.pyapi: the same parameter tables, calls and assertions
on shapes, types, layouts and identities. Where the reference checks no values (its header says so for the fused
operator), the results are compared with numpy or with the oracle here as well."""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cvcuda(cv, gpu):
    return importlib.import_module("cvcuda_amd.pyapi")


RNG = np.random.default_rng(0)


def fill(cvcuda, shape, dtype, layout, rng=RNG, high=None):
    """A tensor with random contents, and the contents."""
    import torch
    dt = np.dtype(dtype)
    if dt.kind == "f":
        a = (rng.random(shape) * (high or 1.0)).astype(dt)
    else:
        a = rng.integers(0, high or min(np.iinfo(dt).max, 1 << 20), shape).astype(dt)
    t = cvcuda.Tensor(shape, dtype, layout)
    view = t.torch()
    src = torch.from_numpy(a.view(np.int16) if dt == np.uint16 else (a.view(np.int32) if dt == np.uint32 else a)).cuda()
    view.copy_(src.view(view.dtype))
    return t, a


def host(tensor):
    import torch
    torch.cuda.synchronize()
    return tensor.torch().cpu().numpy()


def make_batch(cvcuda, n, fmt, size=None, max_size=None, high=None, rng=RNG):
    """n images of `size` (w, h), or of random sizes up to max_size, with random contents; and the contents."""
    import torch
    npdt, ch = cvcuda._PLANE_NP[int(fmt)]
    batch, data = cvcuda.ImageBatchVarShape(n), []
    for _ in range(n):
        w, h = size if size is not None else (int(rng.integers(1, max_size[0] + 1)), int(rng.integers(1, max_size[1] + 1)))
        _, a = None, None
        dt = np.dtype(npdt)
        a = ((rng.random((h, w, ch)) * (high or 1.0)).astype(dt) if dt.kind == "f"
             else rng.integers(0, high or 256, (h, w, ch)).astype(dt))
        img = cvcuda.Image((w, h), fmt)
        img.plane_view(0, dt, ch).copy_(torch.from_numpy(a.view(np.int16) if dt == np.uint16 else a).cuda().view(
            img.plane_view(0, dt, ch).dtype))
        batch.pushback(img)
        data.append(a)
    return batch, data


def clone_batch(cvcuda, batch):
    out = cvcuda.ImageBatchVarShape(batch.capacity)
    out.pushback([cvcuda.Image(img.size, img.format) for img in batch])
    return out


def image_host(cvcuda, img):
    import torch
    npdt, ch = cvcuda._PLANE_NP[int(img.format)]
    torch.cuda.synchronize()
    return img.plane_view(0, npdt, ch).cpu().numpy()


# ---- resize (test_opresize.py:27-139, 198-230) ---------------------------------------------------------------------
@pytest.mark.parametrize("input_args,out_shape,interp", [
    (((5, 16, 23, 4), np.uint8, "NHWC"), (5, 132, 15, 4), "LINEAR"),
    (((16, 23, 4), np.uint8, "HWC"), (132, 15, 4), "CUBIC"),
    (((37, 19, 1), np.uint8, "HWC"), (113, 47, 1), None),
    (((37, 19, 3), np.uint8, "HWC"), (113, 47, 3), "NEAREST"),
    (((37, 19, 1), np.single, "HWC"), (113, 47, 1), None),
    (((37, 19, 3), np.single, "HWC"), (113, 47, 3), None),
])
def test_op_resize(cvcuda, orc, input_args, out_shape, interp):
    interp = None if interp is None else cvcuda.Interp[interp]
    args = () if interp is None else (interp,)
    input, data = fill(cvcuda, *input_args)
    out = cvcuda.resize(input, out_shape, *args)
    assert out.layout == input.layout and out.shape == out_shape and out.dtype == input.dtype
    first = host(out)
    out = cvcuda.Tensor(out_shape, input.dtype, input.layout)
    tmp = cvcuda.resize_into(out, input, *args)
    assert tmp is out
    assert out.layout == input.layout and out.shape == out_shape and out.dtype == input.dtype
    stream = cvcuda.Stream()
    kw = {} if interp is None else {"interp": interp}
    out = cvcuda.resize(src=input, shape=out_shape, stream=stream, **kw)
    stream.sync()
    assert out.layout == input.layout and out.shape == out_shape and out.dtype == input.dtype
    tmp = cvcuda.resize_into(src=input, dst=out, stream=stream, **kw)
    assert tmp is out
    stream.sync()
    np.testing.assert_array_equal(host(out), first)
    # values: the oracle on the same data (default interpolation: LINEAR)
    src4 = data.reshape((1,) * (4 - data.ndim) + data.shape)
    want = orc.resize(src4, (out_shape[-3], out_shape[-2]), int(interp if interp is not None else cvcuda.Interp.LINEAR),
                      variant=1)
    got = first.reshape(want.shape)
    if data.dtype == np.uint8:
        assert np.abs(got.astype(np.int32) - want.astype(np.int32)).max() <= 1
    else:
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("in_shape,out_shape,dtype,interp", [
    ((5, 720, 406, 3), (5, 360, 203, 3), "uint8", "NEAREST"), ((5, 720, 406, 3), (5, 360, 203, 3), "uint8", "LINEAR"),
    ((5, 720, 406, 3), (5, 360, 203, 3), "uint8", "CUBIC"), ((3, 23, 23, 4), (3, 42, 42, 4), "uint8", "LINEAR"),
    ((3, 23, 53, 1), (3, 132, 23, 1), "uint8", "LINEAR"), ((3, 23, 53, 1), (3, 132, 23, 1), "float32", "LINEAR"),
    ((1, 37, 19, 1), (1, 113, 47, 1), "uint8", "LINEAR"), ((1, 37, 19, 3), (1, 113, 47, 3), "uint8", "NEAREST"),
    ((1, 37, 19, 1), (1, 113, 47, 1), "float32", "LINEAR"), ((1, 37, 19, 3), (1, 113, 47, 3), "float32", "LINEAR"),
])
def test_op_resize_packed_torch_tensor(cvcuda, in_shape, out_shape, dtype, interp):
    import torch
    stream = cvcuda.Stream()
    input = torch.empty(in_shape, dtype=getattr(torch, dtype), device="cuda:0")
    output = torch.empty(out_shape, dtype=getattr(torch, dtype), device="cuda:0")
    src = cvcuda.as_tensor(input.cuda(0), "NHWC")
    dst = cvcuda.as_tensor(output.cuda(0), "NHWC")
    tmp = cvcuda.resize_into(dst, src, cvcuda.Interp[interp], stream=stream)
    stream.sync()
    assert tmp is dst
    assert dst.layout == src.layout and dst.shape == out_shape and dst.dtype == src.dtype


@pytest.mark.parametrize("in_size,out_size,interp", [((123, 321), (321, 123), "LINEAR"), ((123, 321), (321, 123), None)])
def test_op_resizevarshape(cvcuda, orc, in_size, out_size, interp):
    input, data = make_batch(cvcuda, 10, cvcuda.Format.RGBA8, size=in_size)
    base_output, _ = make_batch(cvcuda, 10, cvcuda.Format.RGBA8, size=out_size)
    sizes = [[image.width, image.height] for image in base_output]
    args = () if interp is None else (cvcuda.Interp[interp],)
    out = cvcuda.resize(input, sizes, *args)
    assert len(out) == len(base_output) and out.capacity == base_output.capacity
    assert out.uniqueformat == base_output.uniqueformat and out.maxsize == base_output.maxsize
    want = orc.resize(data[3][None], (out_size[1], out_size[0]), 1, variant=1)[0]
    assert np.abs(image_host(cvcuda, out[3]).astype(np.int32) - want.astype(np.int32)).max() <= 1
    stream = cvcuda.Stream()
    tmp = cvcuda.resize_into(src=input, dst=base_output, stream=stream, **({} if interp is None else {"interp": args[0]}))
    assert tmp is base_output
    stream.sync()
    with pytest.raises(RuntimeError):
        cvcuda.resize(input, sizes[:-1])


def test_op_resize_user_stream(cvcuda):
    stream = cvcuda.Stream()
    src = cvcuda.Tensor((5, 1080, 1920, 4), np.uint8, "NHWC")
    with stream:
        assert cvcuda.Stream.current is stream
        dst = cvcuda.resize(src, (5, 108, 192, 4), cvcuda.Interp.NEAREST)
    assert cvcuda.Stream.current is not stream
    stream.sync()
    assert dst.layout == "NHWC" and dst.shape == (5, 108, 192, 4) and dst.dtype == np.uint8


# ---- cvtcolor (test_opcvtcolor.py:24-146) ---------------------------------------------------------------------------
@pytest.mark.parametrize("input_args,code,output_args", [
    ((5, [16, 23], "BGR8"), "BGR2RGB", (5, [16, 23], "RGB8")),
    ((3, [86, 22], "RGBA8"), "RGBA2BGRA", (3, [86, 22], "BGRA8")),
    ((7, [13, 21], "Y8"), "GRAY2BGR", (7, [13, 21], "BGR8")),
    ((9, [66, 99], "HSV8"), "HSV2RGB", (9, [66, 99], "RGB8")),
    (((1, 61, 62, 3), np.uint8, "NHWC"), "YUV2RGB", ((1, 61, 62, 3), np.uint8, "NHWC")),
    (((60, 62, 1), np.uint8, "HWC"), "YUV2RGB_NV12", ((40, 62, 3), np.uint8, "HWC")),
    (((2, 40, 62, 3), np.uint8, "NHWC"), "BGR2YUV_NV21", ((2, 60, 62, 1), np.uint8, "NHWC")),
])
def test_op_cvtcolor(cvcuda, input_args, code, output_args):
    def make(args):
        if isinstance(args[2], str) and hasattr(cvcuda.Format, args[2]) and isinstance(args[0], int):
            return cvcuda.Tensor(args[0], args[1], cvcuda.Format[args[2]])
        return cvcuda.Tensor(*args)
    input, output = make(input_args), make(output_args)
    code = cvcuda.ColorConversion[code]
    out = cvcuda.cvtcolor(input, code)
    assert out.shape == output.shape and out.dtype == output.dtype
    stream = cvcuda.Stream()
    tmp = cvcuda.cvtcolor_into(src=input, dst=output, code=code, stream=stream)
    assert tmp is output
    stream.sync()
    np.testing.assert_array_equal(host(out), host(output))  # both forms ran on the same input


def test_op_cvtcolor_values(cvcuda):
    input, data = fill(cvcuda, (3, 20, 30, 3), np.uint8, "NHWC", high=256)
    np.testing.assert_array_equal(host(cvcuda.cvtcolor(input, cvcuda.ColorConversion.BGR2RGB)), data[..., ::-1])
    rgba = host(cvcuda.cvtcolor(input, cvcuda.ColorConversion.RGB2RGBA))
    np.testing.assert_array_equal(rgba[..., :3], data)
    assert (rgba[..., 3] == 255).all()


@pytest.mark.parametrize("num_images,in_format,img_size,code,out_format", [
    (10, "RGB8", (123, 321), "RGB2RGBA", "RGBA8"), (8, "BGRA8", (23, 21), "BGRA2RGB", "RGB8"),
    (6, "RGB8", (23, 21), "RGB2GRAY", "Y8_ER"), (4, "HSV8", (23, 21), "HSV2RGB", "RGB8"),
    (2, "Y8_ER", (23, 21), "GRAY2BGR", "BGR8"),
])
def test_op_cvtcolorvarshape(cvcuda, num_images, in_format, img_size, code, out_format):
    input, data = make_batch(cvcuda, num_images, cvcuda.Format[in_format], size=img_size, high=256)
    output, _ = make_batch(cvcuda, num_images, cvcuda.Format[out_format], size=img_size, high=256)
    code = cvcuda.ColorConversion[code]
    out = cvcuda.cvtcolor(input, code)
    assert len(out) == len(output) and out.capacity == output.capacity and out.maxsize == output.maxsize
    # codes that share a value (RGB2RGBA = BGR2BGRA ...) give the format of the first name, as in the reference
    assert cvcuda._PLANE_NP[int(out.uniqueformat)] == cvcuda._PLANE_NP[int(output.uniqueformat)]
    stream = cvcuda.Stream()
    tmp = cvcuda.cvtcolor_into(src=input, dst=output, code=code, stream=stream)
    assert tmp is output
    stream.sync()
    for a, b in zip(out, output):
        np.testing.assert_array_equal(image_host(cvcuda, a), image_host(cvcuda, b))
    if in_format == "BGRA8":
        np.testing.assert_array_equal(image_host(cvcuda, out[1]), data[1][..., 2::-1])


# ---- normalize (test_opnormalize.py:24-205) -------------------------------------------------------------------------
@pytest.mark.parametrize("input_args,base_args,scale_args,globalscale,globalshift,epsilon,flags", [
    (((5, 16, 23, 4), np.uint8, "NHWC"), ((1, 1), np.float32, "HW"), ((1, 1), np.float32, "HW"), 1, 2, 3, None),
    (((5, 16, 23, 4), np.uint8, "NHWC"), ((16, 1), np.float32, "HW"), ((16, 1), np.float32, "HW"), 1, 2, 3, "STDDEV"),
    (((5, 16, 23, 4), np.uint8, "NHWC"), ((1, 23), np.float32, "HW"), ((1, 23), np.float32, "HW"), 1, 2, 3, None),
    (((5, 16, 23, 4), np.uint8, "NHWC"), ((16, 23), np.float32, "HW"), ((16, 23), np.float32, "HW"), 1, 2, 3, None),
])
def test_op_normalize(cvcuda, input_args, base_args, scale_args, globalscale, globalshift, epsilon, flags):
    flags = cvcuda.NormalizeFlags.SCALE_IS_STDDEV if flags else None
    input, data = fill(cvcuda, *input_args, high=256)
    base, bdata = fill(cvcuda, *base_args, high=100.0)
    scale, sdata = fill(cvcuda, *scale_args, high=2.0)
    out = cvcuda.normalize(input, base, scale)
    assert out.layout == input.layout and out.shape == input.shape and out.dtype == input.dtype
    want = np.clip(np.rint((data.astype(np.float32) - bdata[None, :, :, None]) * sdata[None, :, :, None]), 0, 255)
    np.testing.assert_array_equal(host(out), want.astype(np.uint8))
    out = cvcuda.Tensor(input.shape, input.dtype, input.layout)
    tmp = cvcuda.normalize_into(out, input, base, scale)
    assert tmp is out
    stream = cvcuda.Stream()
    out = cvcuda.normalize(src=input, base=base, scale=scale, flags=flags, globalscale=globalscale,
                           globalshift=globalshift, epsilon=epsilon, stream=stream)
    assert out.layout == input.layout and out.shape == input.shape and out.dtype == input.dtype
    tmp = cvcuda.normalize_into(src=input, dst=out, base=base, scale=scale, flags=flags, globalscale=globalscale,
                                globalshift=globalshift, epsilon=epsilon, stream=stream)
    assert tmp is out
    stream.sync()


@pytest.mark.parametrize("nimages,format,max_size,max_pixel,base_args,scale_args,globalscale,globalshift,epsilon,flags", [
    (5, "RGB8", (16, 23), 128.0, ((1, 1, 1, 5), np.float32, "NHWC"), ((1, 1, 1, 5), np.float32, "NHWC"), 1, 2, 3, None),
    (5, "RGB8", (16, 23), 256.0, ((1, 1, 1, 5), np.float32, "NHWC"), ((1, 1, 1, 5), np.float32, "NHWC"), 1, 2, 3, "STDDEV"),
])
def test_op_normalizevarshape(cvcuda, nimages, format, max_size, max_pixel, base_args, scale_args, globalscale,
                              globalshift, epsilon, flags):
    flags = cvcuda.NormalizeFlags.SCALE_IS_STDDEV if flags else None
    base, _ = fill(cvcuda, *base_args, high=10.0)
    scale, _ = fill(cvcuda, *scale_args, high=2.0)
    input, _ = make_batch(cvcuda, nimages, cvcuda.Format[format], max_size=max_size, high=int(max_pixel))
    out = cvcuda.normalize(input, base, scale)
    assert len(out) == len(input) and out.capacity == input.capacity
    assert out.uniqueformat == input.uniqueformat and out.maxsize == input.maxsize
    out = clone_batch(cvcuda, input)
    tmp = cvcuda.normalize_into(out, input, base, scale)
    assert tmp is out
    stream = cvcuda.cuda.Stream()
    out = cvcuda.normalize(src=input, base=base, scale=scale, flags=flags, globalscale=globalscale,
                           globalshift=globalshift, epsilon=epsilon, stream=stream)
    assert len(out) == len(input) and out.maxsize == input.maxsize
    tmp = cvcuda.normalize_into(src=input, dst=out, base=base, scale=scale, flags=flags, globalscale=globalscale,
                                globalshift=globalshift, epsilon=epsilon, stream=stream)
    assert tmp is out
    stream.sync()


# ---- reformat, convertto, crops (test_opreformat.py:27-63, test_opconvertto.py:21-60, test_opcustomcrop.py:21-67,
# test_opcentercrop.py:21-48) -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("input_args,out_shape,out_layout", [
    (((5, 16, 23, 4), np.uint8, "NHWC"), (5, 4, 16, 23), "NCHW"), (((5, 16, 23, 3), np.uint8, "NHWC"), (5, 3, 16, 23), "NCHW"),
    (((5, 3, 16, 23), np.uint8, "NCHW"), (5, 16, 23, 3), "NHWC"), (((3, 6, 4), np.uint8, "CHW"), (6, 4, 3), "HWC"),
    (((7, 5, 4), np.uint8, "HWC"), (4, 7, 5), "CHW"),
])
def test_op_reformat(cvcuda, input_args, out_shape, out_layout):
    input, data = fill(cvcuda, *input_args, high=256)
    out = cvcuda.reformat(input, out_layout)
    assert out.layout == out_layout and out.shape == out_shape and out.dtype == input.dtype
    np.testing.assert_array_equal(host(out), data.transpose([input_args[2].index(c) for c in out_layout]))
    out = cvcuda.Tensor(out_shape, input.dtype, out_layout)
    tmp = cvcuda.reformat_into(out, input)
    assert tmp is out
    stream = cvcuda.Stream()
    out = cvcuda.reformat(src=input, layout=out_layout, stream=stream)
    assert out.layout == out_layout and out.shape == out_shape and out.dtype == input.dtype
    tmp = cvcuda.reformat_into(src=input, dst=out, stream=stream)
    assert tmp is out
    stream.sync()


@pytest.mark.parametrize("input_args,dtype,scale,offset", [
    (((5, 16, 23, 4), np.uint8, "NHWC"), np.float32, 1.2, 10.2), (((16, 23, 2), np.uint8, "HWC"), np.int32, -1.2, -5.5),
])
def test_op_convertto(cvcuda, input_args, dtype, scale, offset):
    input, data = fill(cvcuda, *input_args, high=256)
    out = cvcuda.convertto(input, dtype)
    assert out.layout == input.layout and out.shape == input.shape and out.dtype == dtype
    np.testing.assert_array_equal(host(out), data.astype(dtype))
    out = cvcuda.Tensor(input.shape, dtype, input.layout)
    tmp = cvcuda.convertto_into(out, input)
    assert tmp is out
    cvcuda.convertto(input, dtype, scale)
    out = cvcuda.convertto(input, dtype, scale, offset)
    want = data.astype(np.float32) * np.float32(scale) + np.float32(offset)
    if np.dtype(dtype).kind == "f":
        np.testing.assert_allclose(host(out), want, rtol=1e-6)
    else:
        assert np.abs(host(out) - np.rint(want)).max() <= 1
    out = cvcuda.Tensor(input.shape, dtype, input.layout)
    cvcuda.convertto_into(out, input, scale)
    cvcuda.convertto_into(out, input, scale, offset)
    stream = cvcuda.Stream()
    out = cvcuda.convertto(src=input, dtype=dtype, scale=scale, offset=offset, stream=stream)
    assert out.layout == input.layout and out.shape == input.shape and out.dtype == dtype
    tmp = cvcuda.convertto_into(dst=out, src=input, scale=scale, offset=offset, stream=stream)
    assert tmp is out
    stream.sync()


@pytest.mark.parametrize("input_args,rc,out_shape", [
    (((5, 16, 23, 4), np.uint8, "NHWC"), dict(x=0, y=0, width=20, height=2), (5, 2, 20, 4)),
    (((5, 16, 23, 4), np.uint8, "NHWC"), (2, 13, 16, 2), (5, 2, 16, 4)),
    (((16, 23, 2), np.uint8, "HWC"), (2, 13, 16, 2), (2, 16, 2)),
])
def test_op_customcrop(cvcuda, input_args, rc, out_shape):
    rc = cvcuda.RectI(**rc) if isinstance(rc, dict) else cvcuda.RectI(*rc)
    input, data = fill(cvcuda, *input_args, high=256)
    out = cvcuda.customcrop(input, rc)
    assert out.layout == input.layout and out.shape == out_shape and out.dtype == input.dtype
    np.testing.assert_array_equal(host(out), data[..., rc.y:rc.y + rc.height, rc.x:rc.x + rc.width, :])
    out = cvcuda.Tensor(input.shape, input.dtype, input.layout)  # an output larger than the crop is accepted
    tmp = cvcuda.customcrop_into(out, input, rc)
    assert tmp is out and out.shape == input.shape
    stream = cvcuda.Stream()
    out = cvcuda.customcrop(input, rect=rc, stream=stream)
    assert out.layout == input.layout and out.shape == out_shape and out.dtype == input.dtype
    out = cvcuda.Tensor(input.shape, input.dtype, input.layout)
    tmp = cvcuda.customcrop_into(dst=out, src=input, rect=rc, stream=stream)
    assert tmp is out
    stream.sync()


@pytest.mark.parametrize("tensor_args,crop_size,gold_shape", [
    (((5, 9, 9, 4), np.uint8, "NHWC"), [5, 5], (5, 5, 5, 4)), (((9, 9, 3), np.uint8, "HWC"), [5, 5], (5, 5, 3)),
    (((5, 21, 21, 4), np.uint8, "NHWC"), [15, 15], (5, 15, 15, 4)), (((21, 21, 3), np.uint8, "HWC"), [15, 15], (15, 15, 3)),
])
def test_op_center_crop(cvcuda, tensor_args, crop_size, gold_shape):
    input, data = fill(cvcuda, *tensor_args, high=256)
    out = cvcuda.center_crop(input, crop_size)
    assert out.layout == input.layout and out.shape == gold_shape and out.dtype == input.dtype
    h, w = data.shape[-3], data.shape[-2]
    y0, x0 = (h - crop_size[1]) // 2, (w - crop_size[0]) // 2
    np.testing.assert_array_equal(host(out), data[..., y0:y0 + crop_size[1], x0:x0 + crop_size[0], :])
    stream = cvcuda.Stream()
    out = cvcuda.Tensor(input.shape, input.dtype, input.layout)
    tmp = cvcuda.center_crop_into(src=input, dst=out, crop_size=crop_size, stream=stream)
    assert tmp is out and out.shape == input.shape
    stream.sync()


# ---- flip (test_opflip.py:24-131) -----------------------------------------------------------------------------------
@pytest.mark.parametrize("tensor_params,flip_code", [
    (((5, 16, 23, 4), np.uint8, "NHWC"), 0), (((4, 4, 3), np.float32, "HWC"), 1), (((3, 88, 13, 3), np.uint16, "NHWC"), -1),
    (((3, 4, 4), np.int32, "HWC"), 1), (((1, 2, 3, 4), np.uint16, "NHWC"), 0),
])
def test_op_flip(cvcuda, tensor_params, flip_code):
    input, data = fill(cvcuda, *tensor_params)
    out = cvcuda.flip(input, flip_code)
    assert out.layout == input.layout and out.shape == input.shape and out.dtype == input.dtype
    axes = {0: (-3,), 1: (-2,), -1: (-3, -2)}[flip_code]
    np.testing.assert_array_equal(host(out).view(data.dtype), np.flip(data, axes))
    stream = cvcuda.Stream()
    out = cvcuda.Tensor(input.shape, input.dtype, input.layout)
    tmp = cvcuda.flip_into(src=input, dst=out, flipCode=flip_code, stream=stream)
    assert tmp is out
    stream.sync()


@pytest.mark.parametrize("num_images,img_format,img_size,max_pixel", [
    (10, "RGB8", (123, 321), 256), (7, "RGBf32", (62, 35), 1.0), (1, "U16", (33, 48), 1234), (13, "U16", (26, 52), 1234),
    (6, "S32", (77, 42), 123456),
])
def test_op_flipvarshape(cvcuda, num_images, img_format, img_size, max_pixel):
    input, data = make_batch(cvcuda, num_images, cvcuda.Format[img_format], size=img_size, high=max_pixel)
    flipCode, codes = fill(cvcuda, (num_images, 1), np.int32, "NC", high=2)  # 0 or 1 per image
    out = cvcuda.flip(input, flipCode)
    assert len(out) == len(input) and out.capacity == input.capacity
    assert out.uniqueformat == input.uniqueformat and out.maxsize == input.maxsize
    for img, a, code in zip(out, data, codes[:, 0]):
        np.testing.assert_array_equal(image_host(cvcuda, img).view(a.dtype), np.flip(a, 0 if code == 0 else 1))
    stream = cvcuda.Stream()
    out = clone_batch(cvcuda, input)
    tmp = cvcuda.flip_into(src=input, dst=out, flipCode=flipCode, stream=stream)
    assert tmp is out
    stream.sync()


# ---- warps (test_opwarpaffine.py:24-200, test_opwarpperspective.py:24-230) ------------------------------------------
WARP_ROWS = [
    (((5, 16, 23, 4), np.uint8, "NHWC"), [[1, 0, 0], [0, 1, 0]], "NEAREST", "CONSTANT", []),
    (((5, 16, 23, 4), np.uint8, "NHWC"), [[1, 0, 0], [0, 1, 0]], "NEAREST", "CONSTANT", [0]),
    (((5, 16, 23, 4), np.uint8, "NHWC"), [[1, 2, 0], [2, 1, 1]], "LINEAR", "WRAP", [1, 2, 3, 4]),
    (((5, 16, 23, 4), np.uint8, "NHWC"), [[1, 2, 0], [2, 1, 1]], "LINEAR", "REPLICATE", [1, 2, 3, 4]),
    (((11, 21, 4), np.uint8, "HWC"), [[2, 2, 0], [3, 1, 0]], "NEAREST", "CONSTANT", [0]),
    (((11, 21, 4), np.uint8, "HWC"), [[2, 2, 1], [3, 1, 2]], "LINEAR", "WRAP", [1, 2, 3, 4]),
    (((11, 21, 4), np.uint8, "HWC"), [[1, 2, 0], [2, 1, 1]], "LINEAR", "REPLICATE", [1, 2, 3, 4]),
]


@pytest.mark.parametrize("input_args,xform,flags,border_mode,border_value", WARP_ROWS)
@pytest.mark.parametrize("perspective", [False, True])
def test_op_warp(cvcuda, perspective, input_args, xform, flags, border_mode, border_value):
    fn, fn_into = ((cvcuda.warp_perspective, cvcuda.warp_perspective_into) if perspective
                   else (cvcuda.warp_affine, cvcuda.warp_affine_into))
    xform = xform + [[0, 0, 1]] if perspective else xform
    flags, border_mode = cvcuda.Interp[flags], cvcuda.Border[border_mode]
    input, data = fill(cvcuda, *input_args, high=256)
    out = fn(input, xform, flags, border_mode=border_mode, border_value=border_value)
    assert out.layout == input.layout and out.shape == input.shape and out.dtype == input.dtype
    if xform[0][:2] == [1, 0] and xform[1][:2] == [0, 1]:
        np.testing.assert_array_equal(host(out), data)  # the identity map
    stream = cvcuda.Stream()
    out2 = cvcuda.Tensor(input.shape, input.dtype, input.layout)
    tmp = fn_into(src=input, dst=out2, xform=xform, flags=flags, border_mode=border_mode, border_value=border_value,
                  stream=stream)
    assert tmp is out2
    stream.sync()
    np.testing.assert_array_equal(host(out2), host(out))
    with pytest.raises(RuntimeError):
        fn(input, [[1, 0, 0]], flags, border_mode=border_mode, border_value=border_value)


@pytest.mark.parametrize("nimages,format,max_size,max_pixel,max_xval,flags,bmode,border_value", [
    (5, "RGB8", (16, 23), 128, 7, "NEAREST", "CONSTANT", []), (5, "RGB8", (16, 23), 128, 7, "NEAREST", "CONSTANT", [1, 2, 3, 4]),
    (4, "RGB8", (16, 23), 128, 5, "LINEAR", "WRAP", [0]), (3, "RGB8", (16, 23), 128, 4, "CUBIC", "REPLICATE", [2, 1, 0]),
])
@pytest.mark.parametrize("perspective", [False, True])
def test_op_warp_varshape(cvcuda, perspective, nimages, format, max_size, max_pixel, max_xval, flags, bmode, border_value):
    fn, fn_into = ((cvcuda.warp_perspective, cvcuda.warp_perspective_into) if perspective
                   else (cvcuda.warp_affine, cvcuda.warp_affine_into))
    flags, bmode = cvcuda.Interp[flags], cvcuda.Border[bmode]
    input, _ = make_batch(cvcuda, nimages, cvcuda.Format[format], max_size=max_size, high=max_pixel)
    xform, _ = fill(cvcuda, (nimages, 9 if perspective else 6), np.float32, "NC", high=float(max_xval))
    out = fn(input, xform, flags, border_mode=bmode, border_value=border_value)
    assert len(out) == len(input) and out.capacity == input.capacity
    assert out.uniqueformat == input.uniqueformat and out.maxsize == input.maxsize
    stream = cvcuda.Stream()
    out2 = clone_batch(cvcuda, input)
    tmp = fn_into(src=input, dst=out2, xform=xform, flags=flags, border_mode=bmode, border_value=border_value, stream=stream)
    assert tmp is out2
    stream.sync()
    for a, b in zip(out, out2):
        np.testing.assert_array_equal(image_host(cvcuda, a), image_host(cvcuda, b))


# ---- the fused operators (test_opresizecropconvertreformat.py:26-330, test_opcropflipnormalizereformat.py:24-130) ---
RCCR_ROWS = [
    (((4, 512, 512, 3), np.uint8, "NHWC"), (256, 256), "LINEAR", (0, 0, 224, 224), "NCHW", "F32", "REVERSE", (4, 3, 224, 224), 1, 0, True),
    (((4, 512, 512, 3), np.uint8, "NHWC"), (256, 256), "NEAREST", (0, 0, 224, 224), "NCHW", "F32", "REVERSE", (4, 3, 224, 224), 1, 0, True),
    (((4, 512, 512, 3), np.uint8, "NHWC"), (256, 256), "NEAREST", (0, 0, 224, 224), "", "F32", "REVERSE", (4, 224, 224, 3), 1, 0, True),
    (((4, 512, 512, 3), np.uint8, "NHWC"), (256, 256), "NEAREST", (0, 0, 224, 224), "", 0, "REVERSE", (4, 224, 224, 3), 1, 0, True),
    (((17, 678, 1027, 3), np.uint8, "NHWC"), (251, 256), "LINEAR", (0, 0, 200, 22), "NCHW", "F32", "REVERSE", (17, 3, 22, 200), 1, 0, True),
    (((17, 678, 1027, 3), np.uint8, "NHWC"), (251, 256), "LINEAR", (0, 0, 200, 22), "NHWC", "F32", "REVERSE", (17, 22, 200, 3), 1, 0, True),
    (((3, 40, 20, 3), np.uint8, "NHWC"), (160, 160), "NEAREST", (10, 20, 20, 35), "NCHW", "U8", "NO_OP", (3, 3, 35, 20), 1, 0, True),
    (((512, 512, 3), np.uint8, "HWC"), (256, 256), "LINEAR", (0, 0, 224, 224), "CHW", "F32", "REVERSE", (3, 224, 224), 1, 0, True),
    (((3, 512, 512), np.uint8, "CHW"), (256, 256), "LINEAR", (0, 0, 224, 224), "CHW", "F32", "REVERSE", (3, 224, 224), 1, 0, False),
    (((512, 1024, 3), np.uint8, "HWC"), (1024, 256), "LINEAR", (0, 0, 1024, 224), "CHW", "F32", "NO_OP", (3, 224, 1024), 1, 0, True),
    (((4, 678, 1027, 3), np.uint8, "NHWC"), (251, 256), "LINEAR", (0, 0, 200, 22), "NCHW", "F32", "REVERSE", (4, 3, 22, 200), 127.5, -1, True),
    (((512, 1024, 3), np.float32, "HWC"), (1024, 256), "LINEAR", (0, 0, 1024, 224), "CHW", "F32", "REVERSE", (3, 224, 1024), 1, 0, False),
    (((1, 2, 3), np.uint8, "HWC"), (60, 5), "LINEAR", (0, 0, 59, 5), "CHW", "F32", "REVERSE", (3, 5, 59), 1, 0, True),
]


@pytest.mark.parametrize("tensor_params,resize_dim,interp,crop,out_layout,out_dtype,manip,expected,scale,offset,positive",
                         RCCR_ROWS)
def test_op_resize_crop_convert_reformat(cvcuda, orc, tensor_params, resize_dim, interp, crop, out_layout, out_dtype,
                                         manip, expected, scale, offset, positive):
    interp, manip = cvcuda.Interp[interp], cvcuda.ChannelManip[manip]
    out_dtype = cvcuda.Type[out_dtype] if out_dtype else 0
    input, data = fill(cvcuda, *tensor_params, high=256)
    kw = dict(layout=out_layout, data_type=out_dtype, manip=manip, scale=scale, offset=offset)
    if not positive:
        with pytest.raises(Exception):
            cvcuda.resize_crop_convert_reformat(input, resize_dim, interp, cvcuda.RectI(*crop), **kw)
        return
    out = cvcuda.resize_crop_convert_reformat(input, resize_dim, interp, cvcuda.RectI(*crop), **kw)
    assert out.shape == expected
    assert out.layout == (out_layout or input.layout)
    assert out.dtype == (np.dtype(np.float32) if out_dtype == cvcuda.Type.F32 else np.dtype(np.uint8))
    stream = cvcuda.Stream()
    out2 = cvcuda.Tensor(expected, out.dtype, out.layout)
    tmp = cvcuda.resize_crop_convert_reformat_into(out2, input, resize_dim, interp, [crop[0], crop[1]], manip=manip,
                                                  scale=scale, offset=offset, stream=stream)
    assert tmp is out2
    stream.sync()
    np.testing.assert_array_equal(host(out2), host(out))
    # values: the oracle (the reference's own test checks none)
    src4 = data.reshape((1,) * (4 - data.ndim) + data.shape)
    planar = (out_layout or tensor_params[2]).endswith("HW")
    want = orc.fused_rccr(src4, (crop[3], crop[2]), tuple(resize_dim), (crop[0], crop[1]), int(interp),
                          out.dtype.type, planar, int(manip), float(scale), float(offset), True)
    got = host(out).reshape(want.shape)
    if out.dtype == np.uint8:
        assert np.abs(got.astype(np.int32) - want.astype(np.int32)).max() <= 1
    else:
        # srcCast (the default) rounds the interpolated value to u8 first: within 1 LSB of the oracle, times scale
        diff = np.abs(got - want)
        assert diff.max() <= abs(scale) * 1.0001 + 1e-4 and (diff > 1e-4 * max(1.0, abs(scale))).mean() < 0.01


@pytest.mark.parametrize("num_images,min_size,max_size,resize_dim,interp,crop,out_layout,out_dtype,manip,expected", [
    (10, (50, 50), (512, 512), (256, 256), "LINEAR", (0, 0, 224, 224), "NCHW", "F32", "REVERSE", (10, 3, 224, 224)),
    (1, (500, 300), (800, 700), (400, 200), "LINEAR", (0, 0, 224, 190), "NHWC", "F32", "REVERSE", (1, 190, 224, 3)),
    (50, (1, 1), (50, 70), (400, 200), "LINEAR", (0, 0, 224, 190), "NHWC", "F32", "NO_OP", (50, 190, 224, 3)),
    (50, (1, 1), (50, 70), (400, 200), "LINEAR", (0, 0, 224, 190), "NCHW", "U8", "REVERSE", (50, 3, 190, 224)),
    (50, (1, 1), (50, 70), (400, 200), "LINEAR", (0, 0, 224, 190), "NCHW", "U8", "NO_OP", (50, 3, 190, 224)),
    (50, (1, 1), (50, 70), (400, 200), "LINEAR", (0, 0, 224, 190), "", 0, "REVERSE", (50, 190, 224, 3)),
])
def test_op_resize_crop_convert_reformat_varshape(cvcuda, orc, num_images, min_size, max_size, resize_dim, interp, crop,
                                                  out_layout, out_dtype, manip, expected):
    # test_opresizecropconvertreformat.py:262-520
    import torch
    interp, manip = cvcuda.Interp[interp], cvcuda.ChannelManip[manip]
    out_layout = out_layout if out_layout else "NHWC"
    out_dtype = cvcuda.Type[out_dtype] if out_dtype else cvcuda.Type.U8
    input = cvcuda.ImageBatchVarShape(num_images)
    data = []
    for i in range(num_images):
        w = min_size[0] + (max_size[0] - min_size[0]) * i // num_images
        h = min_size[1] + (max_size[1] - min_size[1]) * i // num_images
        a = RNG.integers(0, 256, (h, w, 3)).astype(np.uint8)
        img = cvcuda.Image((w, h), cvcuda.Format.RGB8)
        img.plane_view(0, np.uint8, 3).copy_(torch.from_numpy(a).cuda())
        input.pushback(img)
        data.append(a)
    out1 = cvcuda.resize_crop_convert_reformat(input, resize_dim=resize_dim, interp=interp, crop_rect=cvcuda.RectI(*crop),
                                               layout=out_layout, data_type=out_dtype, manip=manip, scale=1, offset=0)
    assert out1.layout == out_layout and out1.shape == expected and out1.dtype == out_dtype
    out2 = cvcuda.Tensor(expected, out_dtype, out_layout)
    tmp = cvcuda.resize_crop_convert_reformat_into(out2, input, resize_dim, interp, [crop[1], crop[0]], manip=manip)
    assert tmp is out2
    assert out2.layout == out_layout and out2.shape == expected and out2.dtype == out_dtype
    got = host(out1)
    np.testing.assert_array_equal(host(out2), got)
    for i in (0, num_images - 1):  # values: the oracle, within one 8-bit step (the source is cast back to u8 first)
        want = orc.fused_rccr(data[i][None], (crop[3], crop[2]), tuple(resize_dim), (crop[0], crop[1]), int(interp),
                              out1.dtype.type, out_layout == "NCHW", int(manip), 1.0, 0.0, True)
        diff = np.abs(got[i:i + 1].astype(np.float32) - want.astype(np.float32))
        assert diff.max() <= 1.0001 and (diff > 1e-4).mean() < 0.01


@pytest.mark.parametrize("format,num_images,min_size,max_size,border,bvalue,flags,ch,dtype,layout", [
    ("RGBA8", 1, (10, 10), (20, 20), "REPLICATE", 0, "STDDEV", 4, np.uint8, "NHWC"),
    ("RGB8", 4, (10, 12), (30, 24), "CONSTANT", 7, None, 3, np.float32, "NCHW"),
])
def test_op_crop_flip_normalize_reformat(cvcuda, format, num_images, min_size, max_size, border, bvalue, flags, ch, dtype,
                                         layout):
    import torch
    flags = cvcuda.NormalizeFlags.SCALE_IS_STDDEV if flags else None
    border = cvcuda.Border[border]
    base, _ = fill(cvcuda, (1, 1, 1, ch), np.float32, "NHWC", high=10.0)
    scale, _ = fill(cvcuda, (1, 1, 1, ch), np.float32, "NHWC", high=2.0)
    input = cvcuda.ImageBatchVarShape(num_images)
    input.pushback([cvcuda.Image((min_size[0] + (max_size[0] - min_size[0]) * i // num_images,
                                  min_size[1] + (max_size[1] - min_size[1]) * i // num_images), cvcuda.Format[format])
                    for i in range(num_images)])
    for img in input:
        img.plane_view(0, np.uint8, ch).copy_(torch.from_numpy(RNG.integers(0, 256, (img.height, img.width, ch))
                                                                .astype(np.uint8)).cuda())
    # the reference's test leaves the crop rectangles uninitialised; here every image is cropped from its origin
    cropRect = cvcuda.Tensor((num_images, 1, 1, 4), np.int32, "NHWC")
    cropRect.torch().copy_(torch.tensor([[[[0, 0, max_size[1], max_size[0]]]]] * num_images, dtype=torch.int32).cuda())
    flipCode, _ = fill(cvcuda, (num_images, 1), np.int32, "NC", high=2)
    out_shape = (num_images, max_size[0], max_size[1], ch) if layout == "NHWC" else (num_images, ch, max_size[0], max_size[1])
    out = cvcuda.crop_flip_normalize_reformat(input, out_shape, dtype, layout, cropRect, flipCode, base, scale, 1, 2, 3,
                                              flags, border, bvalue)
    assert out.shape == out_shape and out.dtype == dtype and out.layout == layout
    stream = cvcuda.Stream()
    out_tensor = cvcuda.Tensor(out_shape, dtype, layout)
    tmp = cvcuda.crop_flip_normalize_reformat_into(dst=out_tensor, src=input, rect=cropRect, flip_code=flipCode, base=base,
                                                   scale=scale, globalscale=1, globalshift=2, epsilon=3, flags=flags,
                                                   border=border, bvalue=bvalue, stream=stream)
    assert tmp is out_tensor
    stream.sync()
    np.testing.assert_array_equal(host(out_tensor), host(out))


# ---- streams (test_multi_stream.py:21-163) ---------------------------------------------------------------------------
def test_multiple_streams_and_contexts(cvcuda):
    Stream = cvcuda.cuda.Stream
    stream1, stream2, stream3 = Stream(), Stream(), Stream()
    assert stream1 is not stream2 and stream1 is not stream3
    assert Stream.current is Stream.default
    assert Stream.current is not stream1 and Stream.current is not stream2 and Stream.current is not stream3
    with stream1:
        assert Stream.current is stream1
        with stream2:
            assert Stream.current is stream2
        assert Stream.current is stream1
    assert Stream.current is Stream.default
    with pytest.raises(Exception):
        with stream1:
            with stream2:
                assert Stream.current is stream2
                raise Exception()
    assert Stream.current is Stream.default
    with stream2:
        assert Stream.current is stream2
    assert Stream.current is Stream.default


def test_operator_stream(cvcuda):
    import torch
    Stream = cvcuda.cuda.Stream
    for stream in (Stream(), Stream(), Stream()):
        with stream:
            assert Stream.current is stream
            img = cvcuda.as_tensor(torch.zeros(10, 10, 3, dtype=torch.uint8, device="cuda"), "HWC")
            gray = cvcuda.cvtcolor(img, cvcuda.ColorConversion.BGR2GRAY)
            assert gray.shape == (10, 10, 1)
            assert Stream.current is stream
    assert Stream.current is Stream.default


def test_operator_changing_stream(cvcuda):
    # the same two tensors handed from stream to stream: each call must see what the call before it wrote
    import torch
    N, H, W, C, loop = 10, 1080, 1080, 3, 50
    streams = [cvcuda.cuda.Stream() for _ in range(4)]
    input_tensor = torch.randint(0, 256, (N, H, W, C), dtype=torch.uint8).cuda()
    output_tensor = torch.randint(0, 256, (N, H, W, C), dtype=torch.uint8).cuda()
    copy = input_tensor.clone()
    torch.cuda.synchronize()
    tin, tout = cvcuda.as_tensor(input_tensor.data, "NHWC"), cvcuda.as_tensor(output_tensor.data, "NHWC")
    for _ in range(loop):
        for stream in streams:
            cvcuda.flip_into(tout, tin, -1, stream=stream)
            cvcuda.flip_into(tin, tout, -1, stream=stream)
    for stream in streams:
        stream.sync()
    assert torch.equal(torch.as_tensor(tin.cuda(), device="cuda").cpu(), copy.cpu())


def test_operator_changing_stream_loaded(cvcuda):
    # one stream is kept busy; the other takes over the tensors it is still writing
    import torch
    N, H, W, C, loop = 10, 1080, 1080, 3, 6
    stream1, stream2 = cvcuda.cuda.Stream(), cvcuda.cuda.Stream()
    input_tensor = torch.randint(0, 256, (N, H, W, C), dtype=torch.uint8).cuda()
    tmp_tensor = torch.randint(0, 256, (N, H, W, C), dtype=torch.uint8).cuda()
    output_tensor = torch.randint(0, 256, (N, H, W, C), dtype=torch.uint8).cuda()
    copy = input_tensor.clone()
    torch.cuda.synchronize()
    tin, ttmp, tout = (cvcuda.as_tensor(t.data, "NHWC") for t in (input_tensor, tmp_tensor, output_tensor))
    scratch = cvcuda.Tensor((N, H, W, C), np.uint8, "NHWC")
    for _ in range(loop):
        for _ in range(loop * 2):
            cvcuda.flip_into(scratch, ttmp, 0, stream=stream1)
        cvcuda.flip_into(ttmp, tin, -1, stream=stream1)    # ttmp = both axes flipped, behind the busy work
        cvcuda.flip_into(tout, ttmp, -1, stream=stream2)   # reads what stream1 is still writing: tout = tin
        cvcuda.flip_into(tin, tout, 1, stream=stream2)     # tin = columns flipped (stream1 has read tin before)
        cvcuda.flip_into(tout, tin, 1, stream=stream1)     # tout = the original
        cvcuda.flip_into(tin, tout, 0, stream=stream1)     # tin = rows flipped
        cvcuda.flip_into(tout, tin, 0, stream=stream2)     # tout = the original
        cvcuda.flip_into(tin, tout, -1, stream=stream2)    # tin = both flipped
        cvcuda.flip_into(tout, tin, -1, stream=stream1)    # tout = the original
        cvcuda.flip_into(ttmp, tout, 0, stream=stream1)    # ttmp = rows flipped
        cvcuda.flip_into(tin, ttmp, 0, stream=stream2)     # tin = the original again
    stream1.sync()
    stream2.sync()
    assert torch.equal(torch.as_tensor(tin.cuda(), device="cuda").cpu(), copy.cpu())


def test_parallel_callers_share_an_input(cvcuda):
    # after test_multi_threading.py:99-124 (there with an operator outside this path): several threads run an operator
    # on one shared input, each on a stream of its own; every output equals the lone caller's
    import threading
    input, _ = fill(cvcuda, (3, 224, 224, 4), np.uint8, "NHWC", high=256)
    want = host(cvcuda.resize(input, (3, 100, 120, 4), cvcuda.Interp.LINEAR))
    outputs, errors = [], []

    def work():
        try:
            stream = cvcuda.Stream()
            for _ in range(20):
                out = cvcuda.resize(input, (3, 100, 120, 4), cvcuda.Interp.LINEAR, stream=stream)
            stream.sync()
            outputs.append(out)
        except Exception as exc:  # noqa: BLE001 - reported below
            errors.append(repr(exc))

    threads = [threading.Thread(target=work) for _ in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert len(outputs) == 8
    for out in outputs:
        assert out.layout == input.layout and out.dtype == input.dtype
        np.testing.assert_array_equal(host(out), want)


def test_classification_sample_preprocessing(cvcuda, orc):
    # the chain of the reference's classification sample (samples/classification/python/pipelines.py:28-33, 67-90):
    # resize -> convertto(1/255) -> normalize(mean, stddev) -> reformat(NCHW), and the fused operator beside it
    import torch
    frames = torch.randint(0, 256, (4, 360, 640, 3), dtype=torch.uint8).cuda()
    mean_np = np.array([0.485, 0.456, 0.406], np.float32)
    std_np = np.array([0.229, 0.224, 0.225], np.float32)
    mean = cvcuda.as_tensor(torch.from_numpy(mean_np).reshape(1, 1, 1, 3).cuda(), "NHWC")
    stddev = cvcuda.as_tensor(torch.from_numpy(std_np).reshape(1, 1, 1, 3).cuda(), "NHWC")
    out_size = (224, 224)
    frame_nhwc = cvcuda.as_tensor(frames, "NHWC")
    resized = cvcuda.resize(frame_nhwc, (frame_nhwc.shape[0], out_size[1], out_size[0], frame_nhwc.shape[3]),
                            cvcuda.Interp.LINEAR)
    normalized = cvcuda.convertto(resized, np.float32, scale=1 / 255)
    normalized = cvcuda.normalize(normalized, base=mean, scale=stddev, flags=cvcuda.NormalizeFlags.SCALE_IS_STDDEV)
    normalized = cvcuda.reformat(normalized, "NCHW")
    assert normalized.shape == (4, 3, 224, 224) and normalized.dtype == np.float32 and normalized.layout == "NCHW"
    small = host(resized)
    want_small = orc.resize(frames.cpu().numpy(), (224, 224), 1, variant=1)
    assert np.abs(small.astype(np.int32) - want_small.astype(np.int32)).max() <= 1
    unit = small.astype(np.float32) * np.float32(1 / 255)
    want = ((unit - mean_np) * (np.float32(1) / np.sqrt(std_np * std_np))).transpose(0, 3, 1, 2)
    np.testing.assert_allclose(host(normalized), want, rtol=2e-6, atol=2e-6)
    # one call instead of the first two and the last: within one 8-bit step of the chain's unit-range image
    fused = cvcuda.resize_crop_convert_reformat(frame_nhwc, out_size, cvcuda.Interp.LINEAR, cvcuda.RectI(0, 0, 224, 224),
                                                layout="NCHW", data_type=cvcuda.Type.F32, scale=1 / 255)
    assert np.abs(host(fused) - unit.transpose(0, 3, 1, 2)).max() <= 1 / 255 + 1e-6


def test_decoder_and_encoder_edges_of_the_samples(cvcuda, orc, cv):
    # samples/common/python/nvcodec_utils.py:125-137 (decoded NV12 frames -> RGB batch) and :295-316 (NCHW RGB batch
    # -> NHWC -> NV12 for the encoder), with the frames a decoder would hand over replaced by a device buffer
    import importlib.util
    import os
    import torch
    nvcv = cvcuda
    spec = importlib.util.spec_from_file_location("color_oracle_for_pyapi", os.path.join(
        os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "color_oracle.py"))
    col = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(col)
    n, height, width = 3, 96, 128
    surfaces = RNG.integers(16, 236, (n, height * 3 // 2, width, 1)).astype(np.uint8)

    class DecodedFrames:  # what a decoder exposes: device memory through the array interface
        def __init__(self, t):
            self.t = t
            self.__cuda_array_interface__ = t.__cuda_array_interface__

    yuv = nvcv.as_tensor(DecodedFrames(torch.from_numpy(surfaces).cuda()), nvcv.TensorLayout.NHWC)
    rgb_batch = cvcuda.Tensor((n, height, width, 3), nvcv.Type.U8, nvcv.TensorLayout.NHWC)
    cvcuda.cvtcolor_into(rgb_batch, yuv, cvcuda.ColorConversion.YUV2RGB_NV12)
    rgb = host(rgb_batch)
    np.testing.assert_array_equal(rgb, orc.yuv420_to_rgb(surfaces[..., 0], 3, False, 0, True, variant=0))

    # the encoder side: a torch NCHW batch (what the inference side returns) -> NHWC -> NV12
    nchw = torch.from_numpy(rgb.transpose(0, 3, 1, 2).copy()).cuda()
    hwc_batch = cvcuda.Tensor((n, height, width, 3), nvcv.Type.U8, nvcv.TensorLayout.NHWC)
    yuv_batch = cvcuda.Tensor((n, (height // 2) * 3, width, 1), nvcv.Type.U8, nvcv.TensorLayout.NHWC)
    cvcuda.reformat_into(hwc_batch, cvcuda.as_tensor(nchw, nvcv.TensorLayout.NCHW))
    cvcuda.cvtcolor_into(yuv_batch, hwc_batch, cvcuda.ColorConversion.RGB2YUV_NV12)
    tensor = torch.as_tensor(yuv_batch.cuda(), device="cuda")
    torch.cuda.synchronize()
    np.testing.assert_array_equal(host(hwc_batch), rgb)
    np.testing.assert_array_equal(tensor.cpu().numpy().reshape(n, -1, width),
                                  np.asarray(col.yuv420_from_bgr(rgb, False, 0, False)).reshape(n, -1, width))
