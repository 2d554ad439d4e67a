"""The reference's Python interface for the operators of the hot path, on top of this package's classes: the same
function names, argument names, defaults and output-allocation rules as the reference's bindings
(python/mod_cvcuda/Op{Resize,CvtColor,Normalize,Reformat,ConvertTo,CustomCrop,CenterCrop,Flip,WarpAffine,
WarpPerspective,ResizeCropConvertReformat,CropFlipNormalizeReformat}.cpp, CvtColorUtil.cpp:244-330, and the
containers of python/mod_nvcv: Tensor, Image, ImageBatchVarShape, Stream, as_tensor, as_image). A script written
against the reference's `cvcuda` / `nvcv` modules for these operators runs with

    import cvcuda_amd.pyapi as cvcuda
    nvcv = cvcuda

Every function forwards to the C ABI through the operator classes of the package; `stream=None` means the current
stream (`Stream.current`: the innermost `with stream:`, else the default stream). Containers keep the bindings'
ordering across streams: a call on one stream waits for the work of other streams that wrote what it reads or
still uses what it writes. Errors of the C ABI are raised as the
package's `Error`; argument errors the reference's bindings raise themselves (`RuntimeError`, `ValueError`) are
raised as the same types here.
"""
import ctypes as C
import enum
import re
import threading

import numpy as np
import torch

from . import _constants as K
from . import (CenterCrop, ConvertTo, CropFlipNormalizeReformat, CustomCrop, CvtColor, Error, Flip, Normalize, Reformat,
               Resize, ResizeCropConvertReformat, WarpAffine, WarpPerspective)
from . import Image as _Image
from . import ImageBatchVarShape as _ImageBatchVarShape
from . import Tensor as _Tensor
from . import _DT2NP, check
from ._capi import nvcv as _nv

__all__ = ["Error", "Interp", "Border", "ChannelManip", "NormalizeFlags", "ColorConversion", "Format", "Type", "TensorLayout", "RectI",
           "Stream", "as_stream", "cuda", "Tensor", "Image", "ImageBatchVarShape", "as_tensor", "as_image", "as_images", "reshape"]


def _enum_of(name, prefix):
    """Members in the order of the reference's headers: of two names with one value (BGR2BGRA and RGB2RGBA, RGBA2BGR
    and BGRA2RGB ...) the first is the canonical one, as in the reference's table of output formats, where the
    first entry of a value wins (CvtColorUtil.cpp:30-42)."""
    return enum.IntEnum(name, {k[len(prefix):]: v for k, v in vars(K).items()
                               if k.startswith(prefix) and isinstance(v, int)})


class Interp(enum.IntEnum):  # cvcuda/Types.h:39-51
    NEAREST = 0
    LINEAR = 1
    CUBIC = 2
    AREA = 3
    LANCZOS = 4
    GAUSSIAN = 5
    WARP_INVERSE_MAP = 16
    HAMMING = 17
    BOX = 18


class Border(enum.IntEnum):  # nvcv/BorderType.h
    CONSTANT = 0
    REPLICATE = 1
    REFLECT = 2
    WRAP = 3
    REFLECT101 = 4


class ChannelManip(enum.IntEnum):  # cvcuda/Types.h
    NO_OP = 0
    REVERSE = 1


class NormalizeFlags(enum.IntEnum):  # cvcuda/OpNormalize.h
    SCALE_IS_STDDEV = 1


ColorConversion = enum.IntEnum("ColorConversion", {k: int(v) for k, v in _enum_of("_", "COLOR_").__members__.items()
                                                   if re.match(r"^[A-Za-z0-9]+?2[A-Z]", k)})  # not COLOR_SPEC_*, COLOR_XFER_* ...
def _members(prefix):
    """Names of the reference's Python enumerations: the header names without prefix, an underscore in front of
    those that begin with a digit (_2S16, _3S8 ...)."""
    out = {}
    for k, v in vars(K).items():
        if k.startswith(prefix) and isinstance(v, int):
            name = k[len(prefix):]
            out["_" + name if name[0].isdigit() else name] = v
    return out


_nv.nvcvImageFormatGetNumChannels.argtypes = [C.c_uint64, C.POINTER(C.c_int32)]
_nv.nvcvImageFormatGetNumPlanes.argtypes = [C.c_uint64, C.POINTER(C.c_int32)]


class _FormatValue(int):
    @property
    def channels(self):
        n = C.c_int32()
        check(_nv.nvcvImageFormatGetNumChannels(int(self), C.byref(n)))
        return n.value

    @property
    def planes(self):
        n = C.c_int32()
        check(_nv.nvcvImageFormatGetNumPlanes(int(self), C.byref(n)))
        return n.value


_SCALAR_NAMES = {"u1": "U8", "i1": "S8", "u2": "U16", "i2": "S16", "u4": "U32", "i4": "S32", "u8": "U64", "i8": "S64",
                 "f2": "F16", "f4": "F32", "f8": "F64", "c8": "C64", "c16": "C128"}


def _type_name_of(dtype):
    """Member name of Type for a numpy dtype: scalars, and one-dimensional sub-arrays of them ("3i1" -> _3S8)."""
    try:
        dt = np.dtype(dtype)
    except TypeError as exc:
        raise TypeError("not a data type: %r" % (dtype,)) from exc
    count = ""
    if dt.subdtype is not None:
        dt, shape = dt.subdtype
        if len(shape) != 1:
            raise TypeError("only one-dimensional sub-arrays are data types")
        count = "_%d" % shape[0]
    key = dt.kind + str(dt.itemsize)
    if dt.fields is not None or key not in _SCALAR_NAMES:
        raise TypeError("no data type for %r" % (dtype,))
    return count + _SCALAR_NAMES[key]


class _TypeValue(int):
    def __eq__(self, other):
        if isinstance(other, int):
            return int(self) == int(other)
        try:
            return self.name == _type_name_of(other)
        except TypeError:
            return NotImplemented

    def __ne__(self, other):
        result = self.__eq__(other)
        return result if result is NotImplemented else not result

    __hash__ = int.__hash__


Format = enum.Enum("Format", _members("IMAGE_FORMAT_"), type=_FormatValue)


class _TypeMeta(enum.EnumMeta):
    def __call__(cls, value, *args, **kw):
        if not args and not kw and not isinstance(value, int):
            name = _type_name_of(value)
            if name not in cls.__members__:
                raise TypeError("no data type for %r" % (value,))
            return cls.__members__[name]
        return super().__call__(value, *args, **kw)


class _TypeBase(_TypeValue, enum.Enum, metaclass=_TypeMeta):
    """Type(numpy dtype) gives the member; members compare equal to the numpy dtypes they stand for."""


Type = _TypeBase("Type", _members("DATA_TYPE_"))


class TensorLayout:
    """The layout names the reference offers as nvcv.TensorLayout members (python/mod_nvcv/TensorLayout.cpp); a layout
    is passed as its string."""
    NHWC, NCHW, HWC, CHW, NC, NW, NWC, HW, WC, CW, N, C, W = ("NHWC", "NCHW", "HWC", "CHW", "NC", "NW", "NWC", "HW", "WC",
                                                              "CW", "N", "C", "W")


class RectI:
    """x, y, width, height (NVCVRectI)."""

    def __init__(self, x=0, y=0, width=0, height=0):
        self.x, self.y, self.width, self.height = int(x), int(y), int(width), int(height)

    def __iter__(self):
        return iter((self.x, self.y, self.width, self.height))

    def __repr__(self):
        return "RectI(x=%d, y=%d, width=%d, height=%d)" % tuple(self)


# ---- streams -----------------------------------------------------------------------------------------------------
class _StreamMeta(type):
    @property
    def default(cls):
        if cls._default is None:
            cls._default = cls(torch.cuda.default_stream())
        return cls._default

    @property
    def current(cls):
        """The innermost `with stream:` of the calling thread; otherwise the default stream (or torch's current
        stream, when the caller has entered one of torch's stream contexts)."""
        stack = getattr(cls._tls, "stack", None)
        if stack:
            return stack[-1]
        now = torch.cuda.current_stream()
        return cls.default if now == torch.cuda.default_stream() else cls(now)


class Stream(metaclass=_StreamMeta):
    """A HIP stream (python/mod_nvcv/Stream.cpp): `with stream:` makes it the current one of the calling thread."""
    _tls = threading.local()
    _default = None

    def __init__(self, wrapped=None):
        self._s = wrapped if wrapped is not None else torch.cuda.Stream()

    @property
    def handle(self):
        return self._s.cuda_stream

    def __int__(self):
        return self.handle

    def sync(self):
        self._s.synchronize()

    def __enter__(self):
        if not hasattr(self._tls, "stack"):
            self._tls.stack = []
        self._tls.stack.append(self)
        return self

    def __exit__(self, *exc):
        self._tls.stack.pop()
        return False


def as_stream(stream):
    """A Stream over a stream made elsewhere: a torch stream, or a raw hipStream_t given as an int or a
    ctypes.c_void_p (python/mod_nvcv/Stream.cpp, the external-stream wrappers). The wrapper keeps the object."""
    if isinstance(stream, Stream):
        return stream
    if isinstance(stream, C.c_void_p):
        stream = stream.value or 0
    if isinstance(stream, int):
        return Stream.default if stream == 0 else Stream(torch.cuda.ExternalStream(stream))
    if hasattr(stream, "cuda_stream"):
        return Stream(stream)
    raise TypeError("not a stream: %r" % (stream,))


class cuda:  # the reference offers these as cvcuda.cuda.Stream and cvcuda.cuda.as_stream as well
    Stream = Stream
    as_stream = staticmethod(as_stream)


def _torch_stream(stream):
    if stream is None:
        return Stream.current._s
    return stream._s if isinstance(stream, Stream) else stream


# ---- containers --------------------------------------------------------------------------------------------------
def _np_dtype(dtype):
    """numpy dtype of a numpy type, a torch dtype or a member of Type."""
    if isinstance(dtype, (int, enum.IntEnum)) and not isinstance(dtype, bool):
        if int(dtype) not in _DT2NP:
            raise ValueError("data type 0x%x has no array element type" % int(dtype))
        return _DT2NP[int(dtype)]
    if isinstance(dtype, torch.dtype):
        return np.dtype(str(dtype).replace("torch.", ""))
    return np.dtype(dtype)


class _Buffer:
    """What `.cuda()` returns: device memory through `__cuda_array_interface__` and DLPack
    (python/mod_nvcv/ExternalBuffer.cpp)."""

    def __init__(self, iface, owner):
        self.__cuda_array_interface__ = iface
        self._owner = owner
        self.shape = tuple(iface["shape"])
        self.dtype = np.dtype(iface["typestr"])

    @property
    def strides(self):
        """In bytes, as the array interface gives them (dense when it gives none)."""
        given = self.__cuda_array_interface__.get("strides")
        if given is not None:
            return tuple(given)
        out, acc = [], self.dtype.itemsize
        for extent in reversed(self.shape):
            out.insert(0, acc)
            acc *= extent
        return tuple(out)

    def __dlpack__(self, stream=None):
        return torch.as_tensor(self, device="cuda").__dlpack__()

    def __dlpack_device__(self):
        return torch.as_tensor(self, device="cuda").__dlpack_device__()


class Tensor:
    """Tensor(shape, dtype, layout=None) or Tensor(nimages, imgsize=(w, h), format) (python/mod_nvcv/Tensor.cpp)."""

    def __init__(self, *args, rowalign=0, _wrap=None, **kw):
        if _wrap is not None:
            self._t = _wrap
            return
        names = ("nimages", "imgsize", "format") if ("format" in kw or "imgsize" in kw or "nimages" in kw
                                                      or (args and isinstance(args[0], int))) else ("shape", "dtype", "layout")
        vals = dict(zip(names, args))
        vals.update(kw)
        if names[0] == "nimages":
            self._t = _Tensor.for_images(vals["nimages"], tuple(vals["imgsize"]), int(vals["format"]), row_align=rowalign)
        else:
            self._t = _Tensor.alloc(list(vals["shape"]), _np_dtype(vals["dtype"]), vals.get("layout") or "",
                                    row_align=rowalign)

    @property
    def handle(self):
        return self._t.handle

    @property
    def shape(self):
        return tuple(self._t.shape)

    @property
    def ndim(self):
        return len(self._t.shape)

    @property
    def dtype(self):
        return _DT2NP[self._t.dtype]

    @property
    def layout(self):
        return self._t.layout or None

    def cuda(self):
        return _Buffer(self._t.__cuda_array_interface__, self)

    def reshape(self, shape, layout=None):
        return Tensor(_wrap=self._t.reshape(list(shape), layout or ""))

    def torch(self):
        """Strided torch view of the tensor's memory (not in the reference: what its tests build by hand)."""
        return self._t.torch_view()


def reshape(tensor, shape, layout=None):
    """A tensor of another shape over the same memory (nvcvTensorReshape); it keeps the memory alive."""
    return tensor.reshape(shape, layout)


def as_tensor(obj, layout=None):
    """Zero-copy tensor over a torch CUDA tensor, anything with `__cuda_array_interface__` or `__dlpack__`, or an
    image (one image as a tensor of N = 1, nvcvTensorWrapImageConstruct)."""
    if isinstance(obj, _Image):
        handle = C.c_void_p()
        check(_nv.nvcvTensorWrapImageConstruct(obj.handle, C.byref(handle)))
        wrapped = _Tensor(handle)
        wrapped._keep.append(obj)
        return Tensor(_wrap=wrapped)
    if isinstance(obj, torch.Tensor):
        return Tensor(_wrap=_Tensor.from_torch(obj, layout or ""))
    if hasattr(obj, "__cuda_array_interface__"):
        return Tensor(_wrap=_Tensor.from_cuda_array_interface(obj, layout or ""))
    return Tensor(_wrap=_Tensor.from_torch(torch.from_dlpack(obj), layout or ""))


_PLANE_NP = {int(Format.U8): (np.uint8, 1), int(Format.S8): (np.int8, 1), int(Format.U16): (np.uint16, 1),
             int(Format.S16): (np.int16, 1), int(Format.U32): (np.uint32, 1), int(Format.S32): (np.int32, 1),
             int(Format.F32): (np.float32, 1), int(Format.F64): (np.float64, 1), int(Format.Y8): (np.uint8, 1),
             int(Format.Y8_ER): (np.uint8, 1), int(Format.RGB8): (np.uint8, 3), int(Format.BGR8): (np.uint8, 3),
             int(Format.HSV8): (np.uint8, 3), int(Format.RGBA8): (np.uint8, 4), int(Format.BGRA8): (np.uint8, 4),
             int(Format.RGBf32): (np.float32, 3), int(Format.BGRf32): (np.float32, 3),
             int(Format.RGBAf32): (np.float32, 4), int(Format.BGRAf32): (np.float32, 4)}


class Image(_Image):
    """Image(size=(w, h), format) (python/mod_nvcv/Image.cpp)."""

    def __init__(self, size=None, format=None, rowalign=0, *, _handle=None):
        if _handle is None:
            made = _Image.alloc(tuple(size), int(format), row_align=rowalign)
            _handle, made.handle = made.handle, None  # the handle moves to this object
        _Image.__init__(self, _handle)

    @classmethod
    def alloc(cls, size, fmt, base_align=0, row_align=0):
        return cls(size, fmt, rowalign=row_align)

    @classmethod
    def wrap(cls, fmt, planes, keep=None):
        made = _Image.wrap(fmt, planes, keep)
        handle, made.handle = made.handle, None
        img = cls(_handle=handle)
        img._keep.append(keep)
        return img

    @property
    def width(self):
        return self.size[0]

    @property
    def height(self):
        return self.size[1]

    @property
    def format(self):
        value = _Image.format.fget(self)
        try:
            return Format(value)
        except ValueError:
            return value

    @classmethod
    def zeros(cls, size, format, rowalign=0):
        img = cls(size, format, rowalign)
        for buf in img._plane_buffers():
            torch.as_tensor(buf, device="cuda").zero_()
        return img

    def _plane_buffers(self):
        """One (H, W, C) buffer per plane."""
        data = self.export().buffer.strided
        out = []
        for p, (npdt, ch) in enumerate(_planes(int(_Image.format.fget(self)))):
            pl, es = data.planes[p], np.dtype(npdt).itemsize
            iface = {"shape": (pl.height, pl.width, ch), "typestr": np.dtype(npdt).str,
                     "data": (int(pl.basePtr or 0), False), "strides": (pl.rowStride, ch * es, es), "version": 3}
            out.append(_Buffer(iface, self))
        return out

    def cuda(self, layout=None):
        """The image's device memory (python/mod_nvcv/Image.cpp, ExternalBuffer.cpp): one buffer for a packed image
        ((H, W) or (H, W, C)) and for a planar image of equal planes ((C, H, W)), a list of (H, W, C) buffers for
        planes that differ (NV12 ...). `layout` names the dimensions wanted: H, W and C in any order, any other
        letter a dimension of 1."""
        bufs = self._plane_buffers()
        ifaces = [b.__cuda_array_interface__ for b in bufs]
        same = all(i["shape"] == ifaces[0]["shape"] and i["typestr"] == ifaces[0]["typestr"] for i in ifaces)
        if len(bufs) > 1 and not (same and ifaces[0]["shape"][2] == 1):
            return bufs if layout in (None, "HWC") else [_relayout(b, layout) for b in bufs]
        first = ifaces[0]
        h, w, c = first["shape"]
        if len(bufs) > 1:  # equal one-channel planes: C x H x W with the distance of the planes as the C stride
            step = ifaces[1]["data"][0] - first["data"][0]
            merged = dict(first, shape=(len(bufs), h, w), strides=(step, first["strides"][0], first["strides"][2]))
            planar = _Buffer(merged, self)
            return planar if layout in (None, "CHW") else _relayout(planar, layout, have="CHW")
        if layout is None:
            if c == 1:
                return _Buffer(dict(first, shape=(h, w), strides=(first["strides"][0], first["strides"][2])), self)
            return bufs[0]
        return _relayout(bufs[0], layout)

    def cpu(self, layout=None):
        got = self.cuda(layout)
        torch.cuda.synchronize()
        if isinstance(got, list):
            return [torch.as_tensor(g, device="cuda").cpu().numpy() for g in got]
        return torch.as_tensor(got, device="cuda").cpu().numpy()


_nv.nvcvImageFormatGetNumPlanes.argtypes = [C.c_uint64, C.POINTER(C.c_int32)]
_nv.nvcvImageFormatGetPlaneNumChannels.argtypes = [C.c_uint64, C.c_int32, C.POINTER(C.c_int32)]
_nv.nvcvImageFormatGetPlaneDataType.argtypes = [C.c_uint64, C.c_int32, C.POINTER(C.c_uint64)]
_nv.nvcvImageFormatGetPlaneBitsPerPixel.argtypes = [C.c_uint64, C.c_int32, C.POINTER(C.c_int32)]
_nv.nvcvDataTypeGetChannelType.argtypes = [C.c_uint64, C.c_int32, C.POINTER(C.c_uint64)]


def _planes(fmt):
    """(element type, channels) of every plane of an image format."""
    n = C.c_int32()
    check(_nv.nvcvImageFormatGetNumPlanes(fmt, C.byref(n)))
    out = []
    for p in range(n.value):
        ch, dt, el = C.c_int32(), C.c_uint64(), C.c_uint64()
        check(_nv.nvcvImageFormatGetPlaneNumChannels(fmt, p, C.byref(ch)))
        check(_nv.nvcvImageFormatGetPlaneDataType(fmt, p, C.byref(dt)))
        check(_nv.nvcvDataTypeGetChannelType(dt.value, 0, C.byref(el)))
        if el.value not in _DT2NP:
            raise ValueError("plane %d of format 0x%x has no array element type" % (p, fmt))
        # elements per pixel as the memory holds them: bits per pixel / element size (4:2:2 formats such as YUYV
        # name three channels and store two bytes per pixel)
        bpp = C.c_int32()
        check(_nv.nvcvImageFormatGetPlaneBitsPerPixel(fmt, p, C.byref(bpp)))
        out.append((_DT2NP[el.value], max(1, bpp.value // (8 * _DT2NP[el.value].itemsize)) if bpp.value else ch.value))
    return out


def _relayout(buf, layout, have="HWC"):
    """The buffer with its dimensions in the order of `layout`; letters the buffer does not have are dimensions of 1,
    and a dimension the layout leaves out must be 1."""
    iface = buf.__cuda_array_interface__
    dims = dict(zip(have, zip(iface["shape"], iface["strides"])))
    for letter, (extent, _) in dims.items():
        if letter not in layout and extent != 1:
            raise ValueError("layout %r leaves out dimension %s of extent %d" % (layout, letter, extent))
    es = np.dtype(iface["typestr"]).itemsize
    shape = tuple(dims[l][0] if l in dims else 1 for l in layout)
    strides = tuple(dims[l][1] if l in dims else es for l in layout)
    return _Buffer(dict(iface, shape=shape, strides=strides), buf._owner)


def as_image(buffer, format=None):
    """Zero-copy image over an (H, W, C) or (H, W) device buffer; the format is inferred from the element type and
    the channel count when not given (u8 and f32: 1 -> U8 / F32, 3 -> RGB, 4 -> RGBA)."""
    iface, keep = buffer.__cuda_array_interface__, buffer
    shape = tuple(iface["shape"])
    npdt = np.dtype(iface["typestr"])
    if len(shape) == 2:
        shape += (1,)
    if len(shape) != 3:
        raise ValueError("an image buffer has shape (H, W) or (H, W, C)")
    h, w, c = shape
    if format is None:
        table = {(np.dtype(np.uint8), 1): Format.U8, (np.dtype(np.uint8), 3): Format.RGB8,
                 (np.dtype(np.uint8), 4): Format.RGBA8, (np.dtype(np.float32), 1): Format.F32,
                 (np.dtype(np.float32), 3): Format.RGBf32, (np.dtype(np.float32), 4): Format.RGBAf32}
        if (npdt, c) not in table:
            raise ValueError("no image format is inferred for %s x %d" % (npdt, c))
        format = table[(npdt, c)]
    strides = iface.get("strides")
    row = strides[0] if strides else w * c * npdt.itemsize
    return Image.wrap(int(format), [(iface["data"][0], w, h, row)], keep=keep)


def as_images(buffers, format=None):
    """An image batch over a list of (H, W[, C]) device buffers, one image each (capacity = their number)."""
    batch = ImageBatchVarShape(len(buffers))
    batch.pushback([as_image(b, format) for b in buffers])
    return batch


class ImageBatchVarShape(_ImageBatchVarShape):
    """ImageBatchVarShape(capacity) (python/mod_nvcv/ImageBatch.cpp)."""

    def pushback(self, images):
        self.push_back(images)

    def popback(self, count=1):
        self.pop_back(count)

    @property
    def maxsize(self):
        return self.max_size

    @property
    def uniqueformat(self):
        f = self.unique_format
        return Format(f) if f else None

    def __iter__(self):
        return iter(self.images)

    def __getitem__(self, i):
        return self.images[i]


# ---- operators ---------------------------------------------------------------------------------------------------
_ops = {}
_ops_lock = threading.Lock()


def _op(cls, *args):
    with _ops_lock:
        key = (cls,) + args
        if key not in _ops:
            _ops[key] = cls(*args)
        return _ops[key]


def _submit(stream, reads, writes, op, *args):
    """Runs op(stream, *args) with the ordering the reference's bindings give their containers (its ResourceGuard,
    python/mod_nvcv/ResourceGuard.hpp): work on one stream that reads what another stream wrote, or writes what
    another stream still reads or writes, waits for that work first. Each container remembers the event of its last
    write and of the reads since, per stream."""
    s = _torch_stream(stream)
    key = s.cuda_stream
    # the containers' event records are shared by every thread that submits work on them: they are read and
    # updated under one lock (the Submit itself runs outside it)
    with _events_lock:
        waits = []
        for obj in reads + writes:
            wrote = getattr(obj, "_wrote", None)
            if wrote is not None and wrote[0] != key:
                waits.append(wrote[1])
        for obj in writes:
            for other, event in list(getattr(obj, "_read", {}).items()):
                if other != key:
                    waits.append(event)
    for event in waits:
        s.wait_event(event)
    op(s, *args)
    event = _new_event()
    event.record(s)
    with _events_lock:
        for obj in reads:
            obj.__dict__.setdefault("_read", {})[key] = event
        for obj in writes:
            obj._wrote, obj._read = (key, event), {}


_events_lock = threading.Lock()


def _new_event():
    return torch.cuda.Event()


def _same_images(src, fmt=None, sizes=None):
    """A new batch with one image per image of `src`: same sizes and formats unless given."""
    out = ImageBatchVarShape(src.capacity)
    for i, img in enumerate(src.images):
        out.pushback(Image(sizes[i] if sizes is not None else img.size, fmt if fmt is not None else img.format))
    return out


def _image_axes(layout):
    """Positions of W and H in an image tensor layout (None where the layout has none)."""
    if not layout or "W" not in layout:
        raise ValueError("Non-supported tensor layout")
    return layout.index("W"), (layout.index("H") if "H" in layout else None)


def resize_into(dst, src, interp=Interp.LINEAR, *, stream=None):
    _submit(stream, [src], [dst], _op(Resize), src, dst, int(interp))
    return dst


def resize(src, shape=None, interp=Interp.LINEAR, *, sizes=None, stream=None):
    """Tensor: `shape` is the output tensor's shape. Image batch: `sizes` (or the second argument) lists (w, h) per
    image (OpResize.cpp:53-96)."""
    if isinstance(src, _ImageBatchVarShape):
        sizes = sizes if sizes is not None else shape
        if len(src) != len(sizes):
            raise RuntimeError("Number of input images must be equal to the number of elements in output size list ")
        return resize_into(_same_images(src, sizes=[tuple(s) for s in sizes]), src, interp, stream=stream)
    return resize_into(Tensor(tuple(shape), src.dtype, src.layout), src, interp, stream=stream)


_CODE = re.compile(r"^(.*?)2(BGRA|RGBA|BGR|RGB|GRAY|YUV|HSV|HLS|YCrCb|XYZ|Lab|Luv)(.*)$")
_PLANAR_420 = ("_NV12", "_NV21", "_I420", "_IYUV", "_YV12", "420p", "420sp")
_PACKED_422 = ("_UYVY", "_Y422", "_UYNV", "_YUY2", "_YVYU", "_YUYV", "_YUNV")


def _cvtcolor_shape(shape, code):
    """Output tensor shape of a conversion (CvtColorUtil.cpp:281-330: the channel count of the code's output format,
    2/3 or 3/2 of the height for the 4:2:0 codes; in addition, for a 4:2:2 source given with one channel, half the
    width)."""
    if len(shape) not in (3, 4):
        raise RuntimeError("Invalid input tensor shape, only NHWC or HWC are supported")
    m = _CODE.match(ColorConversion(code).name)
    if m is None:
        raise RuntimeError("Invalid color conversion code")
    src, dst, tail = m.groups()
    out = list(shape)
    hi, wi, ci = len(shape) - 3, len(shape) - 2, len(shape) - 1
    to_420 = dst == "YUV" and any(tail.startswith(t) or tail == t.lstrip("_") for t in _PLANAR_420)
    from_420 = src.startswith("YUV") and (any(tail.endswith(t) for t in _PLANAR_420) or src.endswith(("420p", "420sp")))
    from_422 = src.startswith("YUV") and any(tail.endswith(t) for t in _PACKED_422)
    if to_420:
        out[hi], out[ci] = shape[hi] * 3 // 2, 1
    else:
        out[ci] = 4 if dst in ("BGRA", "RGBA") else (1 if dst == "GRAY" else 3)
        if from_420:
            out[hi] = shape[hi] * 2 // 3
        if from_422 and shape[ci] == 1:
            out[wi] = shape[wi] // 2
    return tuple(out)


def _cvtcolor_format(fmt, code):
    """Output image format for a single-plane input format: the code's channel count with the input's element type."""
    npdt, _ = _PLANE_NP[int(fmt)]
    ch = _cvtcolor_shape((1, 1, 1), code)[2]
    name = ColorConversion(code).name
    m = _CODE.match(name)
    dst = m.group(2)
    if np.dtype(npdt) == np.uint8:
        by = {"GRAY": Format.Y8_ER, "HSV": Format.HSV8, "RGB": Format.RGB8, "BGR": Format.BGR8, "RGBA": Format.RGBA8,
              "BGRA": Format.BGRA8, "YUV": Format.YUV8 if ch == 3 else Format.Y8}  # CvtColorUtil.cpp:30-242
        if dst in by:
            return by[dst]
    if np.dtype(npdt) == np.float32:
        by = {"GRAY": Format.F32, "RGB": Format.RGBf32, "BGR": Format.BGRf32, "RGBA": Format.RGBAf32,
              "BGRA": Format.BGRAf32, "HSV": Format.RGBf32}
        if dst in by:
            return by[dst]
    one = {np.dtype(np.uint16): Format.U16, np.dtype(np.int16): Format.S16, np.dtype(np.int32): Format.S32}
    if ch == 1 and np.dtype(npdt) in one:
        return one[np.dtype(npdt)]
    raise RuntimeError("no output image format for %s with %s elements" % (name, np.dtype(npdt)))


def cvtcolor_into(dst, src, code, *, stream=None):
    _submit(stream, [src], [dst], _op(CvtColor), src, dst, int(code))
    return dst


def cvtcolor(src, code, *, stream=None):
    if isinstance(src, _ImageBatchVarShape):
        fmt = src.uniqueformat
        if fmt is None or int(fmt) not in _PLANE_NP:
            raise RuntimeError("All images in input must have the same single-plane format")
        return cvtcolor_into(_same_images(src, fmt=_cvtcolor_format(fmt, code)), src, code, stream=stream)
    layout = "NHWC" if src.ndim == 4 else "HWC"
    return cvtcolor_into(Tensor(_cvtcolor_shape(src.shape, code), src.dtype, layout), src, code, stream=stream)


def normalize_into(dst, src, base, scale, flags=None, *, globalscale=1.0, globalshift=0.0, epsilon=0.0, stream=None):
    _submit(stream, [src, base, scale], [dst], _op(Normalize), src, base, scale, dst, float(globalscale),
            float(globalshift), float(epsilon), int(flags or 0))
    return dst


def normalize(src, base, scale, flags=None, *, globalscale=1.0, globalshift=0.0, epsilon=0.0, stream=None):
    dst = _same_images(src) if isinstance(src, _ImageBatchVarShape) else Tensor(src.shape, src.dtype, src.layout)
    return normalize_into(dst, src, base, scale, flags, globalscale=globalscale, globalshift=globalshift,
                          epsilon=epsilon, stream=stream)


def reformat_into(dst, src, *, stream=None):
    _submit(stream, [src], [dst], _op(Reformat), src, dst)
    return dst


def reformat(src, layout, *, stream=None):
    """The output has the input's dimensions in the order of `layout` (OpReformat.cpp:48-55)."""
    have = src.layout or ""
    if sorted(have) != sorted(layout):
        raise ValueError("layout %r is not a permutation of %r" % (layout, have))
    shape = tuple(src.shape[have.index(c)] for c in layout)
    return reformat_into(Tensor(shape, src.dtype, layout), src, stream=stream)


def convertto_into(dst, src, scale=1, offset=0, *, stream=None):
    _submit(stream, [src], [dst], _op(ConvertTo), src, dst, float(scale), float(offset))
    return dst


def convertto(src, dtype, scale=1, offset=0, *, stream=None):
    return convertto_into(Tensor(src.shape, _np_dtype(dtype), src.layout), src, scale, offset, stream=stream)


def customcrop_into(dst, src, rect, *, stream=None):
    _submit(stream, [src], [dst], _op(CustomCrop), src, dst, tuple(rect))
    return dst


def customcrop(src, rect, *, stream=None):
    wi, hi = _image_axes(src.layout)
    rect = RectI(*rect)
    if hi is None and rect.height != 1:
        raise ValueError("Non-supported tensor layout")
    shape = list(src.shape)
    shape[wi] = rect.width
    if hi is not None:
        shape[hi] = rect.height
    return customcrop_into(Tensor(tuple(shape), src.dtype, src.layout), src, rect, stream=stream)


def center_crop_into(dst, src, crop_size, *, stream=None):
    _submit(stream, [src], [dst], _op(CenterCrop), src, dst, (int(crop_size[0]), int(crop_size[1])))
    return dst


def center_crop(src, crop_size, *, stream=None):
    wi, hi = _image_axes(src.layout)
    if hi is None:
        raise ValueError("Non-supported tensor layout")
    shape = list(src.shape)
    shape[wi], shape[hi] = int(crop_size[0]), int(crop_size[1])
    return center_crop_into(Tensor(tuple(shape), src.dtype, src.layout), src, crop_size, stream=stream)


def flip_into(dst, src, flipCode, *, stream=None):
    """flipCode: an int for tensors; for image batches a tensor with one int32 code per image."""
    if isinstance(src, _ImageBatchVarShape):
        _submit(stream, [src, flipCode], [dst], _op(Flip, src.capacity), src, dst, flipCode)
    else:
        _submit(stream, [src], [dst], _op(Flip, 0), src, dst, int(flipCode))
    return dst


def flip(src, flipCode, *, stream=None):
    dst = _same_images(src) if isinstance(src, _ImageBatchVarShape) else Tensor(src.shape, src.dtype, src.layout)
    return flip_into(dst, src, flipCode, stream=stream)


def _border_value(value):
    v = np.atleast_1d(np.asarray(value, np.float32))
    if v.ndim != 1 or v.size > 4:
        raise RuntimeError("Channels of borderValue should <= 4 and dimension should be 2, current is '%d', '%d' "
                           "respectively" % (v.size, v.ndim))
    return tuple(float(x) for x in v) + (0.0,) * (4 - v.size)


def _matrix(xform, rows):
    m = np.asarray(xform, np.float32)
    if m.ndim != 2 or m.shape != (rows, 3):
        raise RuntimeError("Details of transformation matrix: nDim == 2, shape == (%d, 3) but current is '%d', %s"
                           % (rows, m.ndim, tuple(m.shape)))
    return [float(x) for x in m.reshape(-1)]


def _warp_into(cls, rows, dst, src, xform, flags, border_mode, border_value, stream):
    bv = _border_value(border_value)
    if isinstance(src, _ImageBatchVarShape):
        _submit(stream, [src, xform], [dst], _op(cls, src.capacity), src, dst, xform, int(flags), int(border_mode), bv)
    else:
        _submit(stream, [src], [dst], _op(cls, 0), src, dst, _matrix(xform, rows), int(flags), int(border_mode), bv)
    return dst


def warp_affine_into(dst, src, xform, flags, *, border_mode=Border.CONSTANT, border_value=0, stream=None):
    """xform: a 2 x 3 host array for tensors; for image batches a tensor of N x 6 floats."""
    return _warp_into(WarpAffine, 2, dst, src, xform, flags, border_mode, border_value, stream)


def warp_affine(src, xform, flags, *, border_mode=Border.CONSTANT, border_value=0, stream=None):
    dst = _same_images(src) if isinstance(src, _ImageBatchVarShape) else Tensor(src.shape, src.dtype, src.layout)
    return warp_affine_into(dst, src, xform, flags, border_mode=border_mode, border_value=border_value, stream=stream)


def warp_perspective_into(dst, src, xform, flags, *, border_mode, border_value, stream=None):
    """xform: a 3 x 3 host array for tensors; for image batches a tensor of N x 9 floats."""
    return _warp_into(WarpPerspective, 3, dst, src, xform, flags, border_mode, border_value, stream)


def warp_perspective(src, xform, flags, *, border_mode, border_value, stream=None):
    dst = _same_images(src) if isinstance(src, _ImageBatchVarShape) else Tensor(src.shape, src.dtype, src.layout)
    return warp_perspective_into(dst, src, xform, flags, border_mode=border_mode, border_value=border_value,
                                 stream=stream)


def resize_crop_convert_reformat_into(dst, src, resize_dim, interp, cropPos, *, manip=ChannelManip.NO_OP, scale=1.0,
                                      offset=0.0, srcCast=True, stream=None):
    _submit(stream, [src], [dst], _op(ResizeCropConvertReformat), src, dst, (int(resize_dim[0]), int(resize_dim[1])),
            int(interp), (int(cropPos[0]), int(cropPos[1])), int(manip), float(scale), float(offset), bool(srcCast))
    return dst


def resize_crop_convert_reformat(src, resize_dim, interp, crop_rect, *, layout="", data_type=0,
                                 manip=ChannelManip.NO_OP, scale=1.0, offset=0.0, srcCast=True, stream=None):
    """Output: the input's batch and channels, the crop's height and width, in `layout` (default: the input's) with
    elements of `data_type` (0: the input's). An image batch gives an N-image tensor, `layout` NHWC or NCHW
    (OpResizeCropConvertReformat.cpp:60-103, 132-180)."""
    rect = RectI(*crop_rect)
    if isinstance(src, _ImageBatchVarShape):
        fmt = src.uniqueformat
        if fmt is None or int(fmt) not in _PLANE_NP:
            raise Error(7, "All images in input must have the same single-plane format")
        npdt, ch = _PLANE_NP[int(fmt)]
        src_layout, nhwc = "NHWC", (len(src), rect.height, rect.width, ch)
        src_dtype = np.dtype(npdt)
    else:
        src_layout, src_dtype = src.layout, src.dtype
        if src_layout not in ("HWC", "NHWC"):
            raise Error(7, "Input tensor must have layout 'HWC' or 'NHWC'.")
        shp = (1,) * (4 - src.ndim) + tuple(src.shape)
        nhwc = (shp[0], rect.height, rect.width, shp[3])
    out_layout = layout or src_layout
    if len(out_layout) != len(src_layout):
        raise Error(7, "Output tensor rank must match input tensor rank.")
    if out_layout not in ("HWC", "NHWC", "CHW", "NCHW"):
        raise Error(7, "Output tensor must have layout 'HWC', 'NHWC', 'CHW', or 'NCHW'.")
    shape = tuple(nhwc["NHWC".index(c)] for c in out_layout)
    dst = Tensor(shape, _np_dtype(data_type) if data_type else src_dtype, out_layout)
    return resize_crop_convert_reformat_into(dst, src, resize_dim, interp, (rect.x, rect.y), manip=manip, scale=scale,
                                             offset=offset, srcCast=srcCast, stream=stream)


def crop_flip_normalize_reformat_into(dst, src, rect, flip_code, base, scale, globalscale=1.0, globalshift=0.0,
                                      epsilon=0.0, flags=None, border=Border.CONSTANT, bvalue=0, *, stream=None):
    _submit(stream, [src, rect, flip_code, base, scale], [dst], _op(CropFlipNormalizeReformat), src, dst, rect,
            int(border), float(bvalue), flip_code, base, scale, float(globalscale), float(globalshift), float(epsilon),
            int(flags or 0))
    return dst


def crop_flip_normalize_reformat(src, out_shape, out_dtype, out_layout, rect, flip_code, base, scale, globalscale=1.0,
                                 globalshift=0.0, epsilon=0.0, flags=None, border=Border.CONSTANT, bvalue=0, *,
                                 stream=None):
    dst = Tensor(tuple(out_shape), _np_dtype(out_dtype), out_layout)
    return crop_flip_normalize_reformat_into(dst, src, rect, flip_code, base, scale, globalscale, globalshift, epsilon,
                                             flags, border, bvalue, stream=stream)
