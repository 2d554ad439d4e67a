"""Host-side mirror of the reference's C++ wrapper API (nvcv::Tensor, nvcv::Image,
nvcv::ImageBatchVarShape, cvcuda::<Operator>) on top of this repository's C ABI.

Everything here is a thin ctypes shim: objects own NVCV handles, operators own operator handles,
and each call forwards to the `extern "C"` entry point of the same name. Device memory and streams
come from torch (ROCm build); the arithmetic runs in the HIP kernels inside lib/libcvcuda.so.
Errors are raised as `Error` carrying the NVCVStatus and the library's message.

Reference counterparts: src/nvcv/src/include/nvcv/Tensor.hpp, Image.hpp, ImageBatch.hpp and
src/cvcuda/include/cvcuda/Op*.hpp.
"""
import ctypes as C

import numpy as np
import torch

from . import _capi as capi
from . import _constants as K
from ._capi import cvcuda as _cv
from ._capi import nvcv as _nv


class Error(RuntimeError):
    def __init__(self, status, message):
        super().__init__("%s: %s" % (capi.STATUS_NAMES[status] if 0 <= status < 12 else status, message))
        self.status = status
        self.message = message


def check(status):
    if status != 0:
        buf = C.create_string_buffer(256)
        _nv.nvcvPeekAtLastErrorMessage(buf, 256)
        raise Error(status, buf.value.decode(errors="replace"))


def last_error():
    buf = C.create_string_buffer(256)
    st = _nv.nvcvGetLastErrorMessage(buf, 256)
    return st, buf.value.decode(errors="replace")


# element types ---------------------------------------------------------------------------------
_NP2DT = {
    np.dtype(np.uint8): K.DATA_TYPE_U8, np.dtype(np.int8): K.DATA_TYPE_S8,
    np.dtype(np.uint16): K.DATA_TYPE_U16, np.dtype(np.int16): K.DATA_TYPE_S16,
    np.dtype(np.int32): K.DATA_TYPE_S32, np.dtype(np.uint32): K.DATA_TYPE_U32, np.dtype(np.float32): K.DATA_TYPE_F32,
    np.dtype(np.float64): K.DATA_TYPE_F64, np.dtype(np.float16): K.DATA_TYPE_F16,
    np.dtype(np.complex64): K.DATA_TYPE_C64, np.dtype(np.complex128): K.DATA_TYPE_C128,
}
_DT2NP = {v: k for k, v in _NP2DT.items()}
_NP2TORCH = {
    np.dtype(np.uint8): torch.uint8, np.dtype(np.int8): torch.int8, np.dtype(np.uint16): torch.uint16,
    np.dtype(np.int16): torch.int16, np.dtype(np.int32): torch.int32, np.dtype(np.uint32): torch.uint32,
    np.dtype(np.float32): torch.float32,
    np.dtype(np.float64): torch.float64, np.dtype(np.float16): torch.float16,
    np.dtype(np.complex64): torch.complex64, np.dtype(np.complex128): torch.complex128,
}


def stream_ptr(stream=None):
    """hipStream_t of a torch stream (default: the current one); an int is taken as a raw handle."""
    if isinstance(stream, int):
        return C.c_void_p(stream)
    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


class _DevMem:
    """Exposes raw device memory to torch through the array interface (zero copy)."""

    def __init__(self, ptr, nbytes, owner):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (ptr, False), "version": 2}
        self._owner = owner


def _bytes_view(ptr, nbytes, owner):
    return torch.as_tensor(_DevMem(ptr, nbytes, owner), device="cuda")


class _Handle:
    _pool = None  # "Tensor" | "Image" | "ImageBatch"

    def __init__(self, handle):
        self.handle = C.c_void_p(handle) if not isinstance(handle, C.c_void_p) else handle
        self._keep = []

    def refcount(self):
        n = C.c_int()
        check(getattr(_nv, "nvcv%sRefCount" % self._pool)(self.handle, C.byref(n)))
        return n.value

    def close(self):
        if self.handle is not None and self.handle.value:
            getattr(_nv, "nvcv%sDecRef" % self._pool)(self.handle, None)
        self.handle = None
        self._keep = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Tensor(_Handle):
    _pool = "Tensor"

    # ---- construction ------------------------------------------------------------------------
    @staticmethod
    def requirements(shape, dtype, layout, base_align=0, row_align=0):
        reqs = capi.TensorRequirements()
        shp = (C.c_int64 * len(shape))(*shape)
        check(_nv.nvcvTensorCalcRequirements(len(shape), shp, _as_dtype(dtype), capi.TensorLayout.make(layout),
                                             base_align, row_align, C.byref(reqs)))
        return reqs

    @classmethod
    def alloc(cls, shape, dtype, layout, base_align=0, row_align=0):
        """Library-allocated tensor (hipMalloc through the default allocator)."""
        reqs = cls.requirements(shape, dtype, layout, base_align, row_align)
        h = C.c_void_p()
        check(_nv.nvcvTensorConstruct(C.byref(reqs), None, C.byref(h)))
        return cls(h)

    @classmethod
    def for_images(cls, n, size, fmt, base_align=0, row_align=0):
        reqs = capi.TensorRequirements()
        check(_nv.nvcvTensorCalcRequirementsForImages(n, size[0], size[1], fmt, base_align, row_align,
                                                      C.byref(reqs)))
        h = C.c_void_p()
        check(_nv.nvcvTensorConstruct(C.byref(reqs), None, C.byref(h)))
        return cls(h)

    @classmethod
    def wrap(cls, ptr, shape, strides, dtype, layout, keep=None):
        """Wraps caller-owned device memory (strides in bytes)."""
        d = capi.TensorData()
        d.dtype = _as_dtype(dtype)
        d.layout = capi.TensorLayout.make(layout)
        d.rank = len(shape)
        for i, (s, st) in enumerate(zip(shape, strides)):
            d.shape[i] = s
            d.buffer.strides[i] = st
        d.bufferType = 1
        d.buffer.basePtr = ptr
        h = C.c_void_p()
        check(_nv.nvcvTensorWrapDataConstruct(C.byref(d), None, None, C.byref(h)))
        t = cls(h)
        t._keep.append(keep)
        return t

    @classmethod
    def from_torch(cls, t, layout):
        """Zero-copy view of a torch CUDA tensor."""
        npdt = np.dtype(str(t.dtype).replace("torch.", ""))
        es = t.element_size()
        return cls.wrap(t.data_ptr(), list(t.shape), [s * es for s in t.stride()], npdt, layout, keep=t)

    @classmethod
    def from_cuda_array_interface(cls, obj, layout):
        """Zero-copy view of any object exposing __cuda_array_interface__ (version 2 or 3: CuPy, Numba,
        PyTorch, decoder surfaces ...). The reference offers the same through its external-buffer
        wrapper (python/mod_nvcv/ExternalBuffer.cpp); on ROCm the protocol carries HIP device pointers."""
        iface = obj.__cuda_array_interface__
        npdt = np.dtype(iface["typestr"])
        shape = list(iface["shape"])
        strides = iface.get("strides")
        if strides is None:
            strides, acc = [], npdt.itemsize
            for s_ in reversed(shape):
                strides.insert(0, acc)
                acc *= s_
        return cls.wrap(iface["data"][0], shape, list(strides), npdt, layout, keep=obj)

    @classmethod
    def from_dlpack(cls, obj, layout):
        """Zero-copy view of a DLPack capsule / producer living on this GPU (via torch.utils.dlpack)."""
        return cls.from_torch(torch.utils.dlpack.from_dlpack(obj), layout)

    def to_dlpack(self):
        """DLPack capsule over the tensor's memory; the consumer must not outlive this tensor."""
        return torch.utils.dlpack.to_dlpack(self.torch_view())

    @property
    def __cuda_array_interface__(self):
        d = self.export()
        npdt = _DT2NP[d.dtype]
        return {"shape": tuple(d.shape[i] for i in range(d.rank)), "typestr": npdt.str,
                "data": (int(d.buffer.basePtr or 0), False),
                "strides": tuple(d.buffer.strides[i] for i in range(d.rank)), "version": 3}

    @classmethod
    def from_numpy(cls, a, layout, row_align=0):
        """Uploads a dense host array into a freshly allocated (pitched) tensor."""
        a = np.ascontiguousarray(a)
        t = cls.alloc(list(a.shape), a.dtype, layout, row_align=row_align)
        t.torch_view().copy_(torch.from_numpy(a).cuda())
        return t

    # ---- access --------------------------------------------------------------------------------
    def export(self):
        d = capi.TensorData()
        check(_nv.nvcvTensorExportData(self.handle, C.byref(d)))
        return d

    @property
    def shape(self):
        d = self.export()
        return [d.shape[i] for i in range(d.rank)]

    @property
    def strides(self):
        d = self.export()
        return [d.buffer.strides[i] for i in range(d.rank)]

    @property
    def layout(self):
        return str(self.export().layout)

    @property
    def dtype(self):
        return self.export().dtype

    def torch_view(self):
        """Strided torch view over the tensor's device memory (element type from the tensor dtype)."""
        d = self.export()
        npdt = _DT2NP[d.dtype]
        es = npdt.itemsize
        shape = [d.shape[i] for i in range(d.rank)]
        strides = [d.buffer.strides[i] for i in range(d.rank)]
        nbytes = max(1, sum((s - 1) * st for s, st in zip(shape, strides)) + es)
        raw = _bytes_view(d.buffer.basePtr, nbytes, self)
        if npdt != np.dtype(np.uint8):
            assert all(st % es == 0 for st in strides), "strides must be multiples of the element size"
            raw = raw[: (nbytes // es) * es].view(_NP2TORCH[npdt])
        return torch.as_strided(raw, shape, [st // es for st in strides])

    def numpy(self):
        return self.torch_view().cpu().numpy()

    def reshape(self, shape, layout):
        h = C.c_void_p()
        shp = (C.c_int64 * len(shape))(*shape)
        check(_nv.nvcvTensorReshape(self.handle, len(shape), shp, capi.TensorLayout.make(layout), C.byref(h)))
        t = Tensor(h)
        # the new handle holds a reference on this one, but the owner of externally wrapped memory (a torch tensor,
        # an object with __cuda_array_interface__) is only held by this wrapper: it must live as long as the view
        t._keep.append(self)
        return t


def _as_dtype(dtype):
    if isinstance(dtype, int):
        return dtype
    return _NP2DT[np.dtype(dtype)]


class Image(_Handle):
    _pool = "Image"

    @classmethod
    def alloc(cls, size, fmt, base_align=0, row_align=0):
        reqs = capi.ImageRequirements()
        check(_nv.nvcvImageCalcRequirements(size[0], size[1], fmt, base_align, row_align, C.byref(reqs)))
        h = C.c_void_p()
        check(_nv.nvcvImageConstruct(C.byref(reqs), None, C.byref(h)))
        return cls(h)

    @classmethod
    def wrap(cls, fmt, planes, keep=None):
        """planes: list of (ptr, width, height, rowStride)."""
        d = capi.ImageData()
        d.format = fmt
        d.bufferType = 1
        d.buffer.strided.numPlanes = len(planes)
        for i, (ptr, w, h, rs) in enumerate(planes):
            pl = d.buffer.strided.planes[i]
            pl.basePtr, pl.width, pl.height, pl.rowStride = ptr, w, h, rs
        hh = C.c_void_p()
        check(_nv.nvcvImageWrapDataConstruct(C.byref(d), None, None, C.byref(hh)))
        img = cls(hh)
        img._keep.append(keep)
        return img

    @classmethod
    def from_numpy(cls, a, fmt):
        """Single-plane interleaved image from a dense HxWxC (or HxW) host array."""
        a = np.ascontiguousarray(a)
        img = cls.alloc((a.shape[1], a.shape[0]), fmt)
        img.plane_view(0, a.dtype, a.shape[2] if a.ndim == 3 else 1).copy_(
            torch.from_numpy(a.reshape(a.shape[0], a.shape[1], -1)).cuda())
        return img

    def export(self):
        d = capi.ImageData()
        check(_nv.nvcvImageExportData(self.handle, C.byref(d)))
        return d

    @property
    def size(self):
        w, h = C.c_int32(), C.c_int32()
        check(_nv.nvcvImageGetSize(self.handle, C.byref(w), C.byref(h)))
        return w.value, h.value

    @property
    def format(self):
        f = C.c_uint64()
        check(_nv.nvcvImageGetFormat(self.handle, C.byref(f)))
        return f.value

    def plane_view(self, plane, npdtype, channels):
        """HxWxC strided torch view of one plane."""
        pl = self.export().buffer.strided.planes[plane]
        npdt = np.dtype(npdtype)
        es = npdt.itemsize
        nbytes = (pl.height - 1) * pl.rowStride + pl.width * channels * es
        raw = _bytes_view(pl.basePtr, nbytes, self)
        if npdt != np.dtype(np.uint8):
            raw = raw[: (nbytes // es) * es].view(_NP2TORCH[npdt])
        return torch.as_strided(raw, (pl.height, pl.width, channels), (pl.rowStride // es, channels, 1))


class ImageBatchVarShape(_Handle):
    _pool = "ImageBatch"

    def __init__(self, capacity):
        reqs = capi.ImageBatchVarShapeRequirements()
        check(_nv.nvcvImageBatchVarShapeCalcRequirements(capacity, C.byref(reqs)))
        h = C.c_void_p()
        check(_nv.nvcvImageBatchVarShapeConstruct(C.byref(reqs), None, C.byref(h)))
        super().__init__(h)
        self.images = []

    def push_back(self, images):
        images = list(images) if isinstance(images, (list, tuple)) else [images]
        arr = (C.c_void_p * len(images))(*[i.handle.value for i in images])
        check(_nv.nvcvImageBatchVarShapePushImages(self.handle, arr, len(images)))
        self.images += images

    def pop_back(self, n=1):
        check(_nv.nvcvImageBatchVarShapePopImages(self.handle, n))
        if n:
            del self.images[-n:]

    def clear(self):
        check(_nv.nvcvImageBatchVarShapeClear(self.handle))
        self.images = []

    def __len__(self):
        n = C.c_int32()
        check(_nv.nvcvImageBatchGetNumImages(self.handle, C.byref(n)))
        return n.value

    @property
    def capacity(self):
        n = C.c_int32()
        check(_nv.nvcvImageBatchGetCapacity(self.handle, C.byref(n)))
        return n.value

    @property
    def max_size(self):
        w, h = C.c_int32(), C.c_int32()
        check(_nv.nvcvImageBatchVarShapeGetMaxSize(self.handle, C.byref(w), C.byref(h)))
        return w.value, h.value

    @property
    def unique_format(self):
        f = C.c_uint64()
        check(_nv.nvcvImageBatchVarShapeGetUniqueFormat(self.handle, C.byref(f)))
        return f.value


# operators ---------------------------------------------------------------------------------------
class _Operator:
    _create = None

    def __init__(self, *args):
        h = C.c_void_p()
        check(getattr(_cv, self._create)(C.byref(h), *args))
        self.handle = h

    def close(self):
        if self.handle is not None:
            _cv.nvcvOperatorDestroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _h(obj):
    return obj.handle if obj is not None else None


class ResizeCropConvertReformat(_Operator):
    _create = "cvcudaResizeCropConvertReformatCreate"

    def __call__(self, stream, inp, out, resize_dim, interp, crop_pos, manip=K.CHANNEL_NO_OP, scale=1.0,
                 offset=0.0, src_cast=True):
        fn = (_cv.cvcudaResizeCropConvertReformatVarShapeSubmit if isinstance(inp, ImageBatchVarShape)
              else _cv.cvcudaResizeCropConvertReformatSubmit)
        check(fn(self.handle, stream_ptr(stream), _h(inp), _h(out), capi.Size2D(*resize_dim), interp,
                 capi.Int2(*crop_pos), manip, scale, offset, src_cast))

    def normalized(self, stream, inp, out, resize_dim, interp, crop_pos, base, nscale, manip=K.CHANNEL_NO_OP,
                   scale=1.0, offset=0.0, src_cast=False, global_scale=1.0, shift=0.0, epsilon=0.0, flags=0):
        """Extension: the fused operator followed by a per-channel Normalize in the same kernel."""
        fn = (_cv.cvcudaxResizeCropConvertReformatNormalizeVarShapeSubmit if isinstance(inp, ImageBatchVarShape)
              else _cv.cvcudaxResizeCropConvertReformatNormalizeSubmit)
        nrm = capi.ChannelNormalize((C.c_float * 3)(*base), (C.c_float * 3)(*nscale), global_scale, shift, epsilon,
                                    flags)
        check(fn(self.handle, stream_ptr(stream), _h(inp), _h(out), capi.Size2D(*resize_dim), interp,
                 capi.Int2(*crop_pos), manip, scale, offset, src_cast, C.byref(nrm)))


class Resize(_Operator):
    _create = "cvcudaResizeCreate"

    def __call__(self, stream, inp, out, interp):
        fn = _cv.cvcudaResizeVarShapeSubmit if isinstance(inp, ImageBatchVarShape) else _cv.cvcudaResizeSubmit
        check(fn(self.handle, stream_ptr(stream), _h(inp), _h(out), interp))


class CvtColor(_Operator):
    _create = "cvcudaCvtColorCreate"

    def __call__(self, stream, inp, out, code):
        fn = _cv.cvcudaCvtColorVarShapeSubmit if isinstance(inp, ImageBatchVarShape) else _cv.cvcudaCvtColorSubmit
        check(fn(self.handle, stream_ptr(stream), _h(inp), _h(out), code))


class Normalize(_Operator):
    _create = "cvcudaNormalizeCreate"

    def __call__(self, stream, inp, base, scale, out, global_scale=1.0, shift=0.0, epsilon=0.0, flags=0):
        fn = _cv.cvcudaNormalizeVarShapeSubmit if isinstance(inp, ImageBatchVarShape) else _cv.cvcudaNormalizeSubmit
        check(fn(self.handle, stream_ptr(stream), _h(inp), _h(base), _h(scale), _h(out), global_scale, shift,
                 epsilon, flags))


class Reformat(_Operator):
    _create = "cvcudaReformatCreate"

    def __call__(self, stream, inp, out):
        check(_cv.cvcudaReformatSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out)))


class CropFlipNormalizeReformat(_Operator):
    _create = "cvcudaCropFlipNormalizeReformatCreate"

    def __call__(self, stream, inp, out, crop_rect, border, border_value, flip_code, base, scale, global_scale=1.0,
                 shift=0.0, epsilon=0.0, flags=0):
        check(_cv.cvcudaCropFlipNormalizeReformatSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out),
                                                        _h(crop_rect), border, border_value, _h(flip_code), _h(base),
                                                        _h(scale), global_scale, shift, epsilon, flags))


class ConvertTo(_Operator):
    _create = "cvcudaConvertToCreate"

    def __call__(self, stream, inp, out, alpha=1.0, beta=0.0):
        check(_cv.cvcudaConvertToSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out), alpha, beta))


class CustomCrop(_Operator):
    _create = "cvcudaCustomCropCreate"

    def __call__(self, stream, inp, out, rect):
        """rect: (x, y, width, height)"""
        check(_cv.cvcudaCustomCropSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out), capi.RectI(*rect)))


class CenterCrop(_Operator):
    _create = "cvcudaCenterCropCreate"

    def __call__(self, stream, inp, out, crop_size):
        """crop_size: (width, height)"""
        check(_cv.cvcudaCenterCropSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out), crop_size[0],
                                         crop_size[1]))


class Flip(_Operator):
    _create = "cvcudaFlipCreate"

    def __init__(self, max_varshape_batch_size=0):
        super().__init__(max_varshape_batch_size)

    def __call__(self, stream, inp, out, flip_code):
        """flip_code: int for tensors, an int32 Tensor with one code per image for var-shape batches."""
        if isinstance(inp, ImageBatchVarShape):
            check(_cv.cvcudaFlipVarShapeSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out), _h(flip_code)))
        else:
            check(_cv.cvcudaFlipSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out), flip_code))


class WarpAffine(_Operator):
    _create = "cvcudaWarpAffineCreate"

    def __init__(self, max_varshape_batch_size=0):
        super().__init__(max_varshape_batch_size)

    def __call__(self, stream, inp, out, xform, flags, border=K.BORDER_CONSTANT, border_value=(0, 0, 0, 0)):
        bv = capi.Float4(*[float(v) for v in border_value])
        if isinstance(inp, ImageBatchVarShape):
            check(_cv.cvcudaWarpAffineVarShapeSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out), _h(xform),
                                                     flags, border, bv))
        else:
            m = (C.c_float * 6)(*[float(v) for v in xform])
            check(_cv.cvcudaWarpAffineSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out), m, flags, border, bv))


class WarpPerspective(_Operator):
    _create = "cvcudaWarpPerspectiveCreate"

    def __init__(self, max_varshape_batch_size=0):
        super().__init__(max_varshape_batch_size)

    def __call__(self, stream, inp, out, xform, flags, border=K.BORDER_CONSTANT, border_value=(0, 0, 0, 0)):
        bv = capi.Float4(*[float(v) for v in border_value])
        if isinstance(inp, ImageBatchVarShape):
            check(_cv.cvcudaWarpPerspectiveVarShapeSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out),
                                                          _h(xform), flags, border, bv))
        else:
            m = (C.c_float * 9)(*[float(v) for v in xform])
            check(_cv.cvcudaWarpPerspectiveSubmit(self.handle, stream_ptr(stream), _h(inp), _h(out), m, flags,
                                                  border, bv))
