"""The reference's Python tests of the containers the path's operators take (tests/nvcv_types/python/test_tensor.py:
21-260, test_imgbatchvarshape.py:53-218), restated against cvcuda_amd.pyapi."""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nvcv(cv, gpu):
    return importlib.import_module("cvcuda_amd.pyapi")


@pytest.mark.parametrize("n,size,fmt,gold_layout,gold_shape,gold_dtype", [
    (5, (32, 16), "RGBA8", "NHWC", (5, 16, 32, 4), np.uint8), (2, (38, 7), "RGB8p", "NCHW", (2, 3, 7, 38), np.uint8),
])
def test_tensor_creation_imagebatch_works(nvcv, n, size, fmt, gold_layout, gold_shape, gold_dtype):
    for tensor in (nvcv.Tensor(n, size, nvcv.Format[fmt]), nvcv.Tensor(nimages=n, imgsize=size, format=nvcv.Format[fmt])):
        assert tensor.shape == gold_shape and tensor.layout == gold_layout
        assert tensor.dtype == gold_dtype and tensor.ndim == len(gold_shape)


@pytest.mark.parametrize("shape,dtype,layout", [
    ((5, 16, 32, 4), np.float32, "NHWC"), ((7, 3, 33, 11), np.complex64, "NCHW"), ((3, 11), np.int16, None),
    ((16, 32, 4), np.float32, "HWC"), ((32, 4), np.float32, "WC"), ((4, 32), np.float32, "CW"), ((32,), np.float32, "W"),
])
def test_tensor_creation_shape_works(nvcv, shape, dtype, layout):
    layout = None if layout is None else getattr(nvcv.TensorLayout, layout)
    for tensor in (nvcv.Tensor(shape, dtype, layout), nvcv.Tensor(layout=layout, shape=shape, dtype=dtype)):
        assert tensor.shape == shape and tensor.dtype == dtype and tensor.layout == layout and tensor.ndim == len(shape)


WRAP = [((3, 5, 7, 1), np.uint8), ((3, 5, 7, 1), np.int8), ((3, 5, 7, 1), np.int16), ((3, 5, 7, 1), np.float32),
        ((3, 5, 7, 1), np.float64), ((3, 5, 7, 2), np.float32), ((3, 5, 7, 3), np.uint8), ((3, 5, 7, 4), np.uint8),
        ((3, 5, 7), np.csingle), ((3, 5, 7), np.cdouble), ((3,), np.int8)]


@pytest.mark.parametrize("shape,dtype", WRAP)
@pytest.mark.parametrize("through", ["torch", "dlpack", "cuda_array_interface"])
def test_wrap_torch_buffer(nvcv, shape, dtype, through):
    import torch
    ttensor = torch.as_tensor(np.zeros(shape, dtype=dtype), device="cuda")

    class Only:
        pass
    obj = ttensor
    if through == "dlpack":
        obj = Only()
        obj.__dlpack__, obj.__dlpack_device__ = ttensor.__dlpack__, ttensor.__dlpack_device__
    elif through == "cuda_array_interface":
        obj = Only()
        obj.__cuda_array_interface__ = ttensor.__cuda_array_interface__
    tensor = nvcv.as_tensor(obj)
    assert tensor.shape == shape and tensor.dtype == dtype and tensor.layout is None and tensor.ndim == len(shape)


@pytest.mark.parametrize("shape,dtype,layout", [
    ((3, 5, 7, 1), np.uint8, "NHWC"), ((3, 5, 7), np.uint8, "HWC"), ((3, 5, 7, 2), np.int16, "NHWC"),
    ((3, 5, 7, 2, 4, 2, 5), np.int16, "abcdefg"), ((3, 5), np.uint8, "HW"), ((5,), np.uint8, "W"),
])
def test_wrap_torch_buffer_with_layout(nvcv, shape, dtype, layout):
    import torch
    tensor = nvcv.as_tensor(torch.as_tensor(np.zeros(shape, dtype=dtype), device="cuda"), layout)
    assert tensor.shape == shape and tensor.dtype == dtype and tensor.layout == layout and tensor.ndim == len(shape)


@pytest.mark.parametrize("size,fmt,gold_layout,gold_shape,gold_dtype", [
    ((32, 16), "RGBA8", "NHWC", (1, 16, 32, 4), np.uint8), ((38, 7), "RGB8p", "NCHW", (1, 3, 7, 38), np.uint8),
])
def test_tensor_wrap_image_works(nvcv, size, fmt, gold_layout, gold_shape, gold_dtype):
    img = nvcv.Image(size, nvcv.Format[fmt])
    tensor = nvcv.as_tensor(img)
    assert tensor.shape == gold_shape and tensor.layout == gold_layout and tensor.dtype == gold_dtype


@pytest.mark.parametrize("shape,dtype", [((1, 23, 65, 3), np.uint8), ((5, 23, 65, 3), np.int8), ((65, 3), np.int16),
                                         ((243, 65, 3), np.int16), ((1, 1), np.int16), ((10,), np.uint8)])
def test_tensor_export_cuda_buffer(nvcv, shape, dtype):
    import torch
    gold = np.random.default_rng(1).integers(0, 128, shape, dtype)
    tensor = nvcv.as_tensor(torch.as_tensor(gold, device="cuda"))
    mem = tensor.cuda()
    assert mem.dtype == dtype and mem.shape == shape
    assert (gold == torch.as_tensor(mem, device="cuda").cpu().numpy()).all()
    assert (gold == torch.from_dlpack(mem).cpu().numpy()).all()


def test_tensor_hold_reference_of_wrapped_buffer(nvcv):
    import torch
    ttensor = torch.as_tensor(np.zeros([10], np.int8), device="cuda")
    ptr0 = ttensor.data_ptr()
    cvtensor = nvcv.as_tensor(ttensor)  # noqa: F841 - must keep the first buffer alive
    del ttensor
    ttensor = torch.as_tensor(np.zeros([10], np.int8), device="cuda")
    assert ttensor.data_ptr() != ptr0  # the allocator could not hand the first buffer out again


def test_imgbatchvarshape_creation_works(nvcv):
    batch = nvcv.ImageBatchVarShape(15)
    assert batch.capacity == 15 and len(batch) == 0 and batch.uniqueformat is None and batch.maxsize == (0, 0)
    assert sum(1 for _ in batch) == 0


def test_imgbatchvarshape_one_image(nvcv):
    batch = nvcv.ImageBatchVarShape(15)
    img = nvcv.Image((64, 32), nvcv.Format.RGBA8)
    batch.pushback(img)
    assert len(batch) == 1 and batch.uniqueformat == nvcv.Format.RGBA8 and batch.maxsize == (64, 32)
    assert [b is img for b in batch] == [True]
    batch.popback()
    assert len(batch) == 0 and sum(1 for _ in batch) == 0


def test_imgbatchvarshape_several_images(nvcv):
    batch = nvcv.ImageBatchVarShape(15)
    imgs = [nvcv.Image((m * 2, m), nvcv.Format.RGBA8) for m in range(2, 10, 2)]
    batch.pushback(imgs)
    assert len(batch) == 4 and batch.maxsize == (16, 8) and batch.uniqueformat == nvcv.Format.RGBA8
    assert all(b is i for b, i in zip(batch, imgs)) and sum(1 for _ in batch) == 4
    batch.popback(2)
    assert len(batch) == 2 and sum(1 for _ in batch) == 2 and batch.maxsize == (8, 4)
    batch.pushback(nvcv.Image((58, 26), nvcv.Format.NV12))
    assert batch.maxsize == (58, 26) and batch.uniqueformat is None
    batch.clear()
    assert len(batch) == 0 and sum(1 for _ in batch) == 0 and batch.maxsize == (0, 0)


@pytest.mark.parametrize("base_shape,dt,fmt", [
    ([5, 7, 1], np.uint8, "U8"), ([5, 7], np.uint8, "U8"), ([5, 7, 1], np.float32, "F32"), ([5, 7, 3], np.uint8, "RGB8"),
    ([5, 7, 4], np.uint8, "RGBA8"),
])
def test_wrap_buffer_list(nvcv, base_shape, dt, fmt):
    import torch
    shapes = [[base_shape[d] + (i if d < 2 else 0) for d in range(len(base_shape))] for i in range(3)]
    buffers = [torch.as_tensor(np.zeros(shape, dt), device="cuda") for shape in shapes]
    batch = nvcv.as_images(buffers)
    assert batch.capacity == 3 and batch.maxsize == (base_shape[1] + 2, base_shape[0] + 2)
    assert batch.uniqueformat == nvcv.Format[fmt]
    for image, sh in zip(batch, shapes):
        assert image.width == sh[1] and image.height == sh[0] and image.format == nvcv.Format[fmt]


def test_imgbatchvarshape_wrapper_nodeletion(nvcv):
    import torch
    for i in range(2):
        np_img = np.random.default_rng(i).random((1 + i, 2 + i)).astype(np.float32)
        pt_img = torch.from_numpy(np_img).cuda()
        batch = nvcv.as_images([pt_img])
        del batch
        assert (pt_img.cpu().numpy() == np_img).all()


# ---- images (tests/nvcv_types/python/test_image.py:40-60, 327-445) --------------------------------------------------
def test_image_creation_works(nvcv):
    for img in (nvcv.Image((7, 5), nvcv.Format.NV12), nvcv.Image(size=(7, 5), format=nvcv.Format.NV12)):
        assert img.width == 7 and img.height == 5 and img.size == (7, 5) and img.format == nvcv.Format.NV12


def test_image_create_packed(nvcv):
    import torch
    assert nvcv.Image((37, 11), nvcv.Format.U8, rowalign=1).cuda().__cuda_array_interface__["strides"] == (37, 1)
    assert nvcv.Image.zeros((37, 11), nvcv.Format.U8, rowalign=1).cuda().__cuda_array_interface__["strides"] == (37, 1)
    data = nvcv.as_image(torch.zeros((11, 37), dtype=torch.uint8, device="cuda")).cuda()
    assert data.__cuda_array_interface__["strides"] == (37, 1)
    assert (nvcv.Image.zeros((67, 34), nvcv.Format.F32).cpu() == np.zeros((34, 67), np.float32)).all()


@pytest.mark.parametrize("size,format,layout,out_dtype,out_shape,simple_layout", [
    ((257, 231), "U8", None, np.uint8, (231, 257), "HWC"), ((257, 231), "U8", "HWC", np.uint8, (231, 257, 1), "HWC"),
    ((257, 231), "U8", "CHW", np.uint8, (1, 231, 257), "CHW"),
    ((257, 231), "U8", "xyCrodHlimaWab", np.uint8, (1, 1, 1, 1, 1, 1, 231, 1, 1, 1, 1, 257, 1, 1), "CHW"),
    ((257, 231), "RGBAf32", None, np.float32, (231, 257, 4), "HWC"), ((257, 231), "RGBA8", "HWC", np.uint8, (231, 257, 4), "HWC"),
    ((257, 231), "RGBA8p", None, np.uint8, (4, 231, 257), "CHW"), ((257, 231), "RGBAf32p", "CHW", np.float32, (4, 231, 257), "CHW"),
    ((258, 232), "NV12", None, [np.uint8, np.uint8], [(232, 258, 1), (116, 129, 2)], "HWC"),
    ((258, 232), "NV12", "HWC", [np.uint8, np.uint8], [(232, 258, 1), (116, 129, 2)], "HWC"),
    ((258, 232), "YUYV", None, np.uint8, (232, 258, 2), "HWC"), ((258, 232), "YUYV", "HWC", np.uint8, (232, 258, 2), "HWC"),
])
def test_image_export_cuda_buffer(nvcv, size, format, layout, out_dtype, out_shape, simple_layout):
    import torch
    img = nvcv.Image(size, nvcv.Format[format])
    mem = img.cuda(layout)
    if isinstance(mem, list):
        for m, dt, shp in zip(mem, out_dtype, out_shape):
            assert m.dtype == dt and m.shape == shp
    else:
        assert mem.dtype == out_dtype and mem.shape == out_shape
    assert img.cuda(layout) is not mem  # a buffer is made per call
    buffers = img.cuda(simple_layout)
    buffers = buffers if isinstance(buffers, list) else [buffers]
    rng = np.random.default_rng(0)
    gold = []
    for buf in buffers:  # written on the device side, read back through cpu()
        gold.append((rng.random(size=buf.shape) * 255).astype(buf.dtype))
        torch.as_tensor(buf, device="cuda").copy_(torch.as_tensor(gold[-1]))
    back = img.cpu(simple_layout)
    back = back if isinstance(back, list) else [back]
    for b, g in zip(back, gold):
        np.testing.assert_array_equal(b, g)


# ---- reshape and pitches (test_tensor.py:288-412). Rows are padded to this build's default pitch alignment of 128
# bytes where the reference's figures show its device's 32 ---------------------------------------------------------------
PITCH = 128


def dense(shape):
    out, acc = [], 1
    for extent in reversed(shape):
        out.insert(0, acc)
        acc *= extent
    return tuple(out)


def test_tensor_create_packed(nvcv):
    assert nvcv.Tensor((37, 11, 3), np.uint8, rowalign=1).cuda().strides == (11 * 3, 3, 1)
    assert nvcv.Tensor(2, (37, 7), nvcv.Format.RGB8, rowalign=1).cuda().strides == (37 * 7 * 3, 37 * 3, 3, 1)
    assert nvcv.Tensor((10, 10, 3), np.uint8, layout="HWC").cuda().strides == (PITCH, 3, 1)


@pytest.mark.parametrize("orig_shape,orig_layout,dtype,shape_arg,layout_arg", [
    ((1, 23, 65, 3), "NHWC", np.uint8, (23, 65, 3), "HWC"), ((5, 23, 65, 3), None, np.int8, (5, 23 * 65, 3), None),
    ((5, 23, 65, 3), None, np.int8, (5, 23 * 65, 3), "ABC"), ((1,), "A", np.float32, (1, 1, 1, 1, 1, 1), "ABCDEF"),
])
def test_tensor_reshape(nvcv, orig_shape, orig_layout, dtype, shape_arg, layout_arg):
    tensor = nvcv.Tensor(orig_shape, dtype, layout=orig_layout, rowalign=1)
    es = np.dtype(dtype).itemsize
    assert tensor.dtype == dtype and tensor.shape == orig_shape
    assert tensor.cuda().strides == tuple(s * es for s in dense(orig_shape))
    for new_tensor in (tensor.reshape(shape_arg, layout=layout_arg), nvcv.reshape(tensor, shape_arg, layout=layout_arg)):
        assert new_tensor.dtype == dtype and new_tensor.shape == shape_arg
        assert new_tensor.cuda().strides == tuple(s * es for s in dense(shape_arg))


@pytest.mark.parametrize("orig_shape,orig_layout,dtype,shape_arg,layout_arg", [
    ((1, 23, 65, 3), "NHWC", np.uint8, (23, 65, 3), "ABCD"), ((1, 23, 65, 3), None, np.uint8, (23, 65, 3), "ABCD"),
    ((5, 23, 65, 3), "NHWC", np.int8, (100, 100), "AB"), ((1,), "A", np.int8, tuple(), ""),
])
def test_tensor_reshape_error(nvcv, orig_shape, orig_layout, dtype, shape_arg, layout_arg):
    tensor = nvcv.Tensor(orig_shape, dtype, layout=orig_layout, rowalign=1)
    with pytest.raises(RuntimeError):
        tensor.reshape(shape_arg, layout=layout_arg)
    with pytest.raises(RuntimeError):
        nvcv.reshape(tensor, shape_arg, layout=layout_arg)


def test_tensor_reshape_lifetime_ref_obj(nvcv):
    tensor1 = nvcv.Tensor((20, 10, 3), np.uint8, layout="HWC", rowalign=1)
    tensor2 = tensor1.reshape((200, 3), layout="WC")
    del tensor1  # the reshaped tensor keeps the memory alive
    assert tensor2.dtype == np.uint8 and tensor2.shape == (200, 3) and tensor2.cuda().strides == (3, 1)


@pytest.mark.parametrize("shape_arg,layout_arg,expected_strides", [
    ((1, 10, 10, 3), "XHWC", (10 * PITCH, PITCH, 3, 1)), ((10, 10, 3, 1), "HWCX", (PITCH, 3, 1, 1)),
    ((10, 1, 10, 3), "HXWC", (PITCH, PITCH, 3, 1)), ((10, 2, 5, 3), "HABC", (PITCH, 15, 3, 1)),
    ((2, 5, 10, 3), "ABWC", (5 * PITCH, PITCH, 3, 1)),
])
def test_tensor_reshape_strided(nvcv, shape_arg, layout_arg, expected_strides):
    tensor = nvcv.Tensor((10, 10, 3), np.uint8, layout="HWC")
    assert tensor.cuda().strides == (PITCH, 3, 1)  # padded rows
    for new_tensor in (tensor.reshape(shape_arg, layout=layout_arg), nvcv.reshape(tensor, shape_arg, layout=layout_arg)):
        assert new_tensor.cuda().strides == expected_strides
    with pytest.raises(RuntimeError):  # padded rows cannot become one dense dimension
        tensor.reshape((300,), layout="A")


# ---- streams (tests/nvcv_types/python/test_stream.py:21-112) -----------------------------------------------------------
def test_current_user_and_nested_streams(nvcv):
    Stream = nvcv.cuda.Stream
    assert Stream.current is Stream.default and type(Stream.current) == Stream
    with Stream():
        assert Stream.current is not Stream.default
    stream1, stream2 = Stream(), Stream()
    with stream1:
        assert stream1 is Stream.current and stream1 is not Stream.default
        with stream2:
            assert stream2 is Stream.current and stream1 is not Stream.current
        assert stream2 is not Stream.current and stream1 is Stream.current
    assert stream1 is not Stream.default and stream1 is not Stream.current
    assert Stream.default.handle == 0


def test_wrapped_streams(nvcv):
    import ctypes
    import torch
    stream = torch.cuda.Stream()
    assert nvcv.cuda.as_stream(ctypes.c_void_p(stream.cuda_stream)).handle == stream.cuda_stream
    assert nvcv.cuda.as_stream(int(stream.cuda_stream)).handle == int(stream.cuda_stream)
    own = nvcv.cuda.Stream()
    assert own.handle == int(own)
    ext = torch.cuda.Stream()
    wrapped = nvcv.cuda.as_stream(ext)
    handle = ext.cuda_stream
    assert wrapped.handle == handle
    del ext  # the wrapper keeps the stream alive
    again = nvcv.cuda.as_stream(torch.cuda.ExternalStream(wrapped.handle))
    assert again.handle == handle
    # work submitted on a wrapped stream runs there
    src = nvcv.as_tensor(torch.arange(24, dtype=torch.uint8, device="cuda").reshape(2, 4, 3), "HWC")
    out = nvcv.flip(src, 0, stream=wrapped)
    wrapped.sync()
    assert torch.equal(out.torch().cpu(), torch.arange(24, dtype=torch.uint8).reshape(2, 4, 3).flip(0))
