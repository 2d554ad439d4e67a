"""Host-side rules of cvcuda_amd.pyapi that need no GPU: the enumerations (names that share a value resolve to the
first name of the reference's headers, as its table of output formats does, python/mod_cvcuda/CvtColorUtil.cpp:30-42),
the output shapes and formats of cvtcolor (CvtColorUtil.cpp:244-330) and the argument checks the reference's bindings
make themselves."""
import importlib

import numpy as np
import pytest


@pytest.fixture(scope="module")
def api(cv):
    return importlib.import_module("cvcuda_amd.pyapi")


def test_enumerations(api, K):
    assert api.Interp.LINEAR == K.INTERP_LINEAR and api.Interp.WARP_INVERSE_MAP == K.WARP_INVERSE_MAP == 16
    assert api.Border.REFLECT101 == K.BORDER_REFLECT101 and api.ChannelManip.REVERSE == K.CHANNEL_REVERSE
    assert api.NormalizeFlags.SCALE_IS_STDDEV == 1
    assert api.Format.RGB8 == K.IMAGE_FORMAT_RGB8 and api.Type.F32 == K.DATA_TYPE_F32
    cc = api.ColorConversion
    assert cc.BGR2RGB == K.COLOR_BGR2RGB and cc.YUV2RGB_NV12 == K.COLOR_YUV2RGB_NV12
    assert all("SPEC" not in n and "XFER" not in n for n in cc.__members__)
    # one value, two names: the header's first name is the canonical one
    assert cc.RGB2RGBA is cc.BGR2BGRA and cc(0).name == "BGR2BGRA"
    assert cc.BGRA2RGB is cc.RGBA2BGR and cc(3).name == "RGBA2BGR"


@pytest.mark.parametrize("code,shape,want", [
    ("BGR2GRAY", (2, 8, 6, 3), (2, 8, 6, 1)), ("GRAY2BGR", (8, 6, 1), (8, 6, 3)), ("RGB2RGBA", (8, 6, 3), (8, 6, 4)),
    ("BGRA2RGB", (2, 8, 6, 4), (2, 8, 6, 3)), ("BGR2HSV", (4, 4, 3), (4, 4, 3)), ("BGR2YUV", (8, 6, 3), (8, 6, 3)),
    ("YUV2RGB_NV12", (2, 12, 6, 1), (2, 8, 6, 3)), ("YUV2BGRA_NV21", (60, 62, 1), (40, 62, 4)),
    ("BGR2YUV_NV21", (2, 40, 62, 3), (2, 60, 62, 1)), ("RGB2YUV_NV12", (8, 6, 3), (12, 6, 1)),
    ("YUV2BGR_YUY2", (4, 12, 1), (4, 6, 3)), ("YUV2BGR_YUY2", (4, 6, 2), (4, 6, 3)), ("YUV2GRAY_UYVY", (4, 12, 1), (4, 6, 1)),
])
def test_cvtcolor_output_shapes(api, code, shape, want):
    assert api._cvtcolor_shape(shape, api.ColorConversion[code]) == want


def test_cvtcolor_shape_and_format_errors(api):
    with pytest.raises(RuntimeError):
        api._cvtcolor_shape((8, 6), api.ColorConversion.BGR2RGB)
    F, cc = api.Format, api.ColorConversion
    assert api._cvtcolor_format(F.RGB8, cc.RGB2GRAY) == F.Y8_ER and api._cvtcolor_format(F.Y8, cc.GRAY2BGR) == F.BGR8
    assert api._cvtcolor_format(F.HSV8, cc.HSV2RGB) == F.RGB8 and api._cvtcolor_format(F.BGRA8, cc.BGRA2RGB) == F.BGR8
    assert api._cvtcolor_format(F.RGB8, cc.RGB2YUV_NV12) == F.Y8 and api._cvtcolor_format(F.BGRf32, cc.RGB2BGR) == F.RGBf32  # = BGR2RGB


def test_small_helpers(api):
    r = api.RectI(x=1, y=2, width=3, height=4)
    assert tuple(r) == (1, 2, 3, 4) and tuple(api.RectI(5, 6, 7, 8)) == (5, 6, 7, 8)
    assert api._border_value([]) == (0.0, 0.0, 0.0, 0.0) and api._border_value(3) == (3.0, 0.0, 0.0, 0.0)
    assert api._border_value([1, 2, 3, 4]) == (1.0, 2.0, 3.0, 4.0)
    with pytest.raises(RuntimeError):
        api._border_value([1, 2, 3, 4, 5])
    assert api._matrix([[1, 0, 2], [0, 1, 3]], 2) == [1.0, 0.0, 2.0, 0.0, 1.0, 3.0]
    with pytest.raises(RuntimeError):
        api._matrix([[1, 0, 2]], 2)
    assert api._image_axes("NHWC") == (2, 1) and api._image_axes("CHW") == (2, 1) and api._image_axes("NWC") == (1, None)
    with pytest.raises(ValueError):
        api._image_axes("NC")
    assert api._np_dtype(api.Type.F32) == np.float32 and api._np_dtype(np.uint8) == np.uint8


# ---- tests/nvcv_types/python/test_imgformat.py:20-45, test_datatype.py:21-54, test_rect.py:19-40 ------------------------
@pytest.mark.parametrize("format,gold_channels,gold_planes", [
    ("RGBA8", 4, 1), ("RGB8", 3, 1), ("_2S16", 2, 1), ("S8", 1, 1), ("NV12", 3, 2),
])
def test_imgformat_numchannels_and_planes(api, format, gold_channels, gold_planes):
    assert getattr(api.Format, format).channels == gold_channels and getattr(api.Format, format).planes == gold_planes


@pytest.mark.parametrize("type,dt", [
    ("U8", np.uint8), ("U8", np.dtype(np.uint8)), ("S8", np.int8), ("U16", np.uint16), ("S16", np.int16), ("U32", np.uint32),
    ("S32", np.int32), ("U64", np.uint64), ("S64", np.int64), ("F32", np.float32), ("F64", np.float64), ("C64", np.complex64),
    ("_2C64", np.dtype("2F")), ("C128", np.complex128), ("_2C128", np.dtype("2D")), ("_3S8", np.dtype("3i1")),
    ("_4S32", np.dtype("4i")),
])
def test_datatype_dtype(api, type, dt):
    type = getattr(api.Type, type)
    assert type == dt
    made = api.Type(dt)
    assert made == type and made == dt and made is type


@pytest.mark.parametrize("dt", [np.dtype([("f1", np.uint64), ("f2", np.int32)]), "invalid"])
def test_datatype_dtype_conv_error(api, dt):
    with pytest.raises(TypeError):
        api.Type(dt)


def test_recti(api):
    r = api.RectI()
    assert (r.x, r.y, r.width, r.height) == (0, 0, 0, 0)
    for x, y, w, h in ((0, 0, 0, 0), (10, -12, -45, 14)):
        for r in (api.RectI(x, y, w, h), api.RectI(y=y, width=w, height=h, x=x)):
            assert (r.x, r.y, r.width, r.height) == (x, y, w, h)


def test_reshape_of_wrapped_memory_keeps_its_owner_alive(api):
    # nvcvTensorReshape takes a reference on the source handle, but the owner of externally wrapped memory is held by the
    # Python wrapper of the source only: the reshaped tensor must hold it too (no GPU: the pointer is never followed)
    import gc
    import weakref

    class Owner:
        def __init__(self):
            self.__cuda_array_interface__ = {"shape": (8, 3, 3), "typestr": "|u1", "data": (0x7F0000001000, False),
                                             "version": 3, "strides": None}

    owner = Owner()
    alive = weakref.ref(owner)
    source = api.as_tensor(owner, "HWC")
    for view in (source.reshape((24, 3), "WC"), api.reshape(source, (72,), "W")):
        del source, owner
        gc.collect()
        assert alive() is not None, "the owner of the wrapped memory was collected while a reshaped tensor refers to it"
        assert view.cuda().__cuda_array_interface__["data"][0] == 0x7F0000001000
        owner = alive()
        source = api.as_tensor(owner, "HWC")
        del view
    del source, owner
    gc.collect()
    assert alive() is None


def test_submit_bookkeeping_under_parallel_readers(api, monkeypatch):
    # several threads record reads of one shared input on their own streams while another thread keeps writing it:
    # no read event may be lost (a later writer waits for every stream that read) and no iteration may trip over a
    # concurrent update. No GPU: streams and events are stand-ins that only record what was asked of them.
    import threading

    class FakeStream:
        def __init__(self, key):
            self.cuda_stream, self.waited = key, []

        def wait_event(self, event):
            self.waited.append(event)

    class FakeEvent:
        def record(self, stream):
            self.stream = stream.cuda_stream

    class Box:
        pass

    monkeypatch.setattr(api, "_torch_stream", lambda s: s)
    monkeypatch.setattr(api, "_new_event", FakeEvent)
    shared, errors = Box(), []

    def reader(key):
        try:
            out = Box()
            for _ in range(300):
                api._submit(FakeStream(key), [shared], [out], lambda s: None)
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=reader, args=(100 + i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert sorted(shared._read) == [100 + i for i in range(8)]
    writer = FakeStream(7)
    api._submit(writer, [], [shared], lambda s: None)
    assert sorted(e.stream for e in writer.waited) == [100 + i for i in range(8)]
    assert shared._read == {} and shared._wrote[0] == 7
