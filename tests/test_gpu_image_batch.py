"""Life cycle of a variable-shape image batch on the GPU, following the reference's own unit tests
(tests/nvcv_types/system/TestImageBatch.cpp:74-358, 552-600): what the exported descriptor lists on the device hold
after pushes, pops and a push of a second format, and that rewriting the batch on the host right after an export
does not disturb the upload that export started."""
import ctypes as C
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def fields(buf):
    """The meaningful fields of an NVCVImageBufferStrided (padding and unused planes left out)."""
    return (buf.numPlanes,) + tuple((p.width, p.height, p.rowStride, p.basePtr)
                                    for p in list(buf.planes)[:buf.numPlanes])


def strided_of(capi, img):
    d = img.export()
    assert d.bufferType == 1  # NVCV_IMAGE_BUFFER_STRIDED_CUDA
    return fields(d.buffer.strided), d.format


def export(cv, capi, batch, stream):
    data = capi.ImageBatchData()
    cv.check(capi.nvcv.nvcvImageBatchExportData(batch.handle, C.c_void_p(stream), C.byref(data)))
    assert data.bufferType == 1  # NVCV_IMAGE_BATCH_VARSHAPE_BUFFER_STRIDED_CUDA
    return data


def device_lists(cv, capi, torch, data, stream):
    """Reads the device-side image and format lists back on `stream`."""
    n = data.numImages
    sz = C.sizeof(capi.ImageBufferStrided)
    with torch.cuda.stream(stream):
        imgs = cv._bytes_view(data.buffer.imageList, max(n, 1) * sz, None).cpu()
        fmts = cv._bytes_view(data.buffer.formatList, max(n, 1) * 8, None).cpu()
    stream.synchronize()
    raw = imgs.numpy().tobytes()
    bufs = [fields(capi.ImageBufferStrided.from_buffer_copy(raw[i * sz:(i + 1) * sz])) for i in range(n)]
    return bufs, list(np.frombuffer(fmts.numpy().tobytes(), np.uint64)[:n])


def host_formats(data):
    return list((C.c_uint64 * data.numImages).from_address(data.buffer.hostFormatList)) if data.numImages else []


def test_descriptor_lists_follow_pushes_pops_and_formats(cv, K, gpu):
    import torch
    capi = __import__("sys").modules["cvcuda_amd._capi"]
    nv = capi.nvcv
    stream = torch.cuda.Stream()
    batch = cv.ImageBatchVarShape(100)
    assert batch.capacity == 100 and len(batch) == 0
    ty = C.c_int(-1)
    assert nv.nvcvImageBatchGetType(batch.handle, C.byref(ty)) == 0 and ty.value == 0  # NVCV_TYPE_IMAGEBATCH_VARSHAPE

    data = export(cv, capi, batch, 0)
    assert data.numImages == 0 and data.buffer.imageList and data.buffer.formatList
    assert (data.buffer.maxWidth, data.buffer.maxHeight) == (0, 0) == batch.max_size
    assert data.buffer.uniqueFormat == K.IMAGE_FORMAT_NONE == batch.unique_format

    gold = []

    def push(images):
        batch.push_back(images)
        gold.extend(images if isinstance(images, list) else [images])

    def max_size():
        return (max(i.size[0] for i in gold), max(i.size[1] for i in gold))

    push(cv.Image.alloc((320, 128), K.IMAGE_FORMAT_NV12))
    push([cv.Image.alloc((320, 128), K.IMAGE_FORMAT_NV12)])
    first = [cv.Image.alloc((328 + i * 2, 130 - i * 2), K.IMAGE_FORMAT_NV12) for i in range(10)]
    push(first)
    push([cv.Image.alloc((328 + i * 2, 130 - i * 2), K.IMAGE_FORMAT_NV12) for i in range(10)])
    data = export(cv, capi, batch, stream.cuda_stream)
    assert (data.buffer.maxWidth, data.buffer.maxHeight) == max_size() == batch.max_size

    push([cv.Image.alloc((328 + i * 2, 130 - i * 2), K.IMAGE_FORMAT_NV12) for i in range(10)])
    push(first)  # the same images may be in a batch twice
    batch.pop_back(5)
    del gold[-5:]
    data = export(cv, capi, batch, stream.cuda_stream)
    assert (data.buffer.maxWidth, data.buffer.maxHeight) == max_size() == batch.max_size
    assert data.buffer.uniqueFormat == K.IMAGE_FORMAT_NV12 == batch.unique_format
    assert host_formats(data) == [K.IMAGE_FORMAT_NV12] * len(gold)

    push(cv.Image.alloc((42, 59), K.IMAGE_FORMAT_RGBA8))  # a second format: no unique format any more
    data = export(cv, capi, batch, stream.cuda_stream)
    assert data.buffer.uniqueFormat == K.IMAGE_FORMAT_NONE == batch.unique_format
    assert data.numImages == len(gold) == len(batch)
    assert (data.buffer.maxWidth, data.buffer.maxHeight) == max_size() == batch.max_size
    want = [strided_of(capi, i) for i in gold]
    images, formats = device_lists(cv, capi, torch, data, stream)
    assert images == [w[0] for w in want]
    assert formats == [w[1] for w in want] == host_formats(data)

    out = (C.c_void_p * len(gold))()
    assert nv.nvcvImageBatchVarShapeGetImages(batch.handle, 0, out, len(gold)) == 0
    assert list(out) == [i.handle.value for i in gold]
    for h in out:
        assert nv.nvcvImageDecRef(C.c_void_p(h), None) == 0  # each handle handed out carries a reference

    # popping the odd format brings the unique format back
    batch.pop_back(1)
    assert batch.unique_format == K.IMAGE_FORMAT_NV12

    up = C.c_void_p(1)
    assert nv.nvcvImageBatchGetUserPointer(batch.handle, C.byref(up)) == 0 and up.value is None
    assert nv.nvcvImageBatchSetUserPointer(batch.handle, C.c_void_p(0x123)) == 0
    assert nv.nvcvImageBatchGetUserPointer(batch.handle, C.byref(up)) == 0 and up.value == 0x123
    n = C.c_int()
    assert nv.nvcvImageBatchIncRef(batch.handle, C.byref(n)) == 0 and n.value == 2
    assert nv.nvcvImageBatchDecRef(batch.handle, C.byref(n)) == 0 and n.value == 1


def test_rewriting_the_batch_after_an_export_does_not_disturb_the_upload(cv, K, gpu):
    import torch
    capi = __import__("sys").modules["cvcuda_amd._capi"]
    stream = torch.cuda.Stream()
    rng = random.Random(123)
    capacity = 4000
    batch = cv.ImageBatchVarShape(capacity)
    # all images live in two slabs, wrapped: thousands of separate device allocations would only slow the test
    slab = torch.empty(2 * capacity * 8 * 16, dtype=torch.uint8, device=gpu)

    def make(k):
        w, h = rng.randint(1, 4) * 2, rng.randint(1, 4) * 2
        base = slab.data_ptr() + k * 128
        return cv.Image.wrap(K.IMAGE_FORMAT_NV12, [(base, w, h, 8), (base + 64, w // 2, h // 2, 8)])

    first = [make(k) for k in range(capacity)]
    second = [make(capacity + k) for k in range(capacity)]
    want = [strided_of(capi, i)[0] for i in first]
    batch.push_back(first)
    data = export(cv, capi, batch, stream.cuda_stream)  # starts the host -> device copy on `stream`
    batch.clear()
    batch.push_back(second)                              # rewrites the host mirror: must wait for that copy
    assert data.numImages == capacity
    images, _ = device_lists(cv, capi, torch, data, stream)
    assert images == want
    # the next export uploads the new contents
    data = export(cv, capi, batch, stream.cuda_stream)
    images, _ = device_lists(cv, capi, torch, data, stream)
    assert images == [strided_of(capi, i)[0] for i in second]
