"""Edge cases shared by the operators: empty image batches, one-pixel images, rows whose width is not
a multiple of anything, odd base addresses and pitches (views into a larger buffer)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

NEAREST, LINEAR, CUBIC, AREA = 0, 1, 2, 3


def test_empty_image_batches_are_rejected_like_the_reference(cv, K, gpu):
    # nothing pushed: a batch without images has no format, which the reference reports as
    # INVALID_ARGUMENT (e.g. legacy/resize_var_shape.cu:502-506); nothing is launched
    a, b = cv.ImageBatchVarShape(4), cv.ImageBatchVarShape(4)
    ident = cv.Tensor.from_numpy(np.tile(np.array([[1, 0, 0, 0, 1, 0]], np.float32), (4, 1)), "NW")
    codes = cv.Tensor.from_numpy(np.zeros(4, np.int32), "N")
    one = cv.Tensor.from_numpy(np.ones((1, 1, 1, 1), np.float32), "NHWC")
    calls = [lambda: cv.Resize()(None, a, b, LINEAR),
             lambda: cv.WarpAffine(4)(None, a, b, ident, LINEAR, 0, (0, 0, 0, 0)),
             lambda: cv.Flip(4)(None, a, b, codes),
             lambda: cv.Normalize()(None, a, one, one, b),
             lambda: cv.CvtColor()(None, a, b, K.COLOR_BGR2RGB)]
    for call in calls:
        with pytest.raises(cv.Error) as e:
            call()
        assert e.value.status == 2
    torch.cuda.synchronize()
    assert len(a) == 0 and len(b) == 0


@pytest.mark.parametrize("dt,c", [(np.uint8, 1), (np.uint8, 3), (np.uint8, 4), (np.uint16, 3), (np.float32, 1),
                                  (np.float32, 4)])
def test_one_pixel_and_one_row_images(cv, orc, gpu, dt, c):
    rng = np.random.default_rng(11)
    for (sh, sw), (dh, dw) in [((1, 1), (1, 1)), ((1, 1), (5, 7)), ((1, 9), (1, 4)), ((9, 1), (4, 1)), ((1, 9), (3, 13)),
                               ((2, 2), (5, 5)), ((3, 3), (1, 1))]:
        src = (rng.random((2, sh, sw, c)) * 200).astype(dt)
        for interp in (NEAREST, LINEAR, CUBIC):
            out = cv.Tensor.alloc([2, dh, dw, c], dt, "NHWC")
            cv.Resize()(None, cv.Tensor.from_numpy(src, "NHWC"), out, interp)
            torch.cuda.synchronize()
            ref = orc.resize_shipped(src, (dh, dw), interp)
            got = out.numpy()
            if dt == np.float32:
                assert np.abs(got - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max()), (sh, sw, dh, dw, interp)
            else:
                np.testing.assert_array_equal(got, ref, err_msg=str((sh, sw, dh, dw, interp)))


def test_odd_base_addresses_and_pitches(cv, K, orc, gpu):
    # operators on views that start at an odd byte of a larger buffer and have an odd row pitch: the
    # run kernels' dword accesses must not assume alignment
    n, h, w, c = 2, 19, 37, 3
    pitch, plane = w * c + 5, (w * c + 5) * h + 3
    src = orc.fill_u8((n, h, w, c), 77)
    big_in = torch.zeros(n * plane + 64, dtype=torch.uint8, device="cuda")
    big_out = torch.full((n * plane + 64,), 0xCD, dtype=torch.uint8, device="cuda")
    view_in = torch.as_strided(big_in[1:], (n, h, w, c), (plane, pitch, c, 1))
    view_in.copy_(torch.from_numpy(src).cuda())

    def wrap(buf, elem=1, ch=c):
        return cv.Tensor.wrap(buf.data_ptr() + 1, [n, h, w, ch], [plane, pitch, ch * elem, elem], np.uint8, "NHWC", keep=buf)

    tin, tout = wrap(big_in), wrap(big_out)
    out_view = torch.as_strided(big_out[1:], (n, h, w, c), (plane, pitch, c, 1))

    def untouched():
        mask = torch.ones_like(big_out, dtype=torch.bool)
        torch.as_strided(mask[1:], (n, h, w * c), (plane, pitch, 1)).fill_(False)
        return bool((big_out[mask] == 0xCD).all())

    cv.CvtColor()(None, tin, tout, K.COLOR_BGR2RGB)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out_view.cpu().numpy(), src[..., ::-1])
    assert untouched()

    cv.Flip()(None, tin, tout, 1)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out_view.cpu().numpy(), src[:, :, ::-1])
    assert untouched()

    base = cv.Tensor.from_numpy(np.array([[[[3.0, 5.0, 7.0]]]], np.float32), "NHWC")
    scale = cv.Tensor.from_numpy(np.array([[[[0.5, 1.5, 2.0]]]], np.float32), "NHWC")
    cv.Normalize()(None, tin, base, scale, tout, 1.0, 0.0, 0.0, 0)
    torch.cuda.synchronize()
    ref = orc.normalize(src, np.array([[[[3.0, 5.0, 7.0]]]], np.float32), np.array([[[[0.5, 1.5, 2.0]]]], np.float32))
    np.testing.assert_array_equal(out_view.cpu().numpy(), ref)
    assert untouched()

    cv.Resize()(None, tin, tout, LINEAR)  # same size: identity
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out_view.cpu().numpy(), src)
    assert untouched()

    ident = [1, 0, 0, 0, 1, 0]
    cv.WarpAffine(0)(None, tin, tout, ident, LINEAR, 0, (0, 0, 0, 0))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out_view.cpu().numpy(), src)
    assert untouched()


def test_submits_captured_in_a_hip_graph_replay_correctly(cv, K, orc, gpu):
    # a pipeline of Submits (fused resize -> Normalize -> Reformat, plus a warp) is captured once and
    # replayed with new input contents and eager work in between; every replay must equal the eager result
    n = 3
    tin = cv.Tensor.alloc([n, 90, 160, 3], np.uint8, "NHWC")
    t1 = cv.Tensor.alloc([n, 32, 32, 3], np.float32, "NHWC")
    t2 = cv.Tensor.alloc([n, 32, 32, 3], np.float32, "NHWC")
    t3 = cv.Tensor.alloc([n, 3, 32, 32], np.float32, "NCHW")
    tw = cv.Tensor.alloc([n, 90, 160, 3], np.uint8, "NHWC")
    base = cv.Tensor.from_numpy(np.array([[[[0.4, 0.5, 0.6]]]], np.float32), "NHWC")
    scale = cv.Tensor.from_numpy(np.array([[[[0.2, 0.3, 0.4]]]], np.float32), "NHWC")
    fused, norm, ref_, warp = cv.ResizeCropConvertReformat(), cv.Normalize(), cv.Reformat(), cv.WarpAffine(0)
    mat = [0.9, -0.2, 7.0, 0.2, 0.9, -3.0]

    def pipeline(stream):
        fused(stream, tin, t1, (64, 36), LINEAR, (16, 2), 0, 1 / 255.0, 0.0, False)
        norm(stream, t1, base, scale, t2, 1.0, 0.0, 0.0, K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV)
        ref_(stream, t2, t3)
        warp(stream, tin, tw, mat, LINEAR, 0, (0, 0, 0, 0))

    tin.torch_view().copy_(torch.from_numpy(orc.fill_u8((n, 90, 160, 3), 1)).cuda())
    pipeline(torch.cuda.current_stream())  # warm up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pipeline(torch.cuda.current_stream())
    for seed in (2, 3, 4):
        src = orc.fill_u8((n, 90, 160, 3), seed)
        tin.torch_view().copy_(torch.from_numpy(src).cuda())
        t3.torch_view().zero_()
        tw.torch_view().zero_()
        graph.replay()
        torch.cuda.synchronize()
        got3, gotw = t3.numpy().copy(), tw.numpy().copy()
        t3.torch_view().zero_()
        tw.torch_view().zero_()
        pipeline(torch.cuda.current_stream())  # eager work between the replays
        torch.cuda.synchronize()
        np.testing.assert_array_equal(got3, t3.numpy())
        np.testing.assert_array_equal(gotw, tw.numpy())
        x = orc.fused_rccr(src, (32, 32), (64, 36), (16, 2), LINEAR, np.float32, False, 0, 1 / 255.0, 0.0, False)
        want = orc.normalize(x, np.array([[[[0.4, 0.5, 0.6]]]], np.float32), np.array([[[[0.2, 0.3, 0.4]]]], np.float32),
                             1.0, 0.0, 0.0, True).transpose(0, 3, 1, 2)
        assert (np.abs(got3 - want) <= 1e-5 * np.maximum(1.0, np.abs(want))).all()


def test_image_batch_descriptors_must_be_uploaded_before_graph_capture(cv, K, orc, gpu):
    # A var-shape Submit uploads the descriptors of images pushed since the last Submit on the caller's stream.
    # Under graph capture that copy would be recorded into the graph (and replay whatever the host mirror holds
    # later), so it is refused with INVALID_OPERATION; after one Submit outside the capture the same call captures.
    imgs = [orc.fill_u8((20 + 2 * i, 30 + i, 3), 40 + i) for i in range(3)]
    bi, bo, outs = cv.ImageBatchVarShape(3), cv.ImageBatchVarShape(3), []
    for a in imgs:
        bi.push_back(cv.Image.from_numpy(a, K.IMAGE_FORMAT_RGB8))
        outs.append(cv.Image.alloc((a.shape[1], a.shape[0]), K.IMAGE_FORMAT_RGB8))
        bo.push_back(outs[-1])
    op = cv.CvtColor()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        with pytest.raises(cv.Error) as e:
            op(torch.cuda.current_stream(), bi, bo, K.COLOR_BGR2RGB)
    assert e.value.status == 4  # NVCV_ERROR_INVALID_OPERATION
    op(None, bi, bo, K.COLOR_BGR2RGB)  # uploads the descriptors
    torch.cuda.synchronize()
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph2, stream=side):
        op(torch.cuda.current_stream(), bi, bo, K.COLOR_BGR2RGB)
    graph2.replay()
    torch.cuda.synchronize()
    for a, o in zip(imgs, outs):
        np.testing.assert_array_equal(o.plane_view(0, np.uint8, 3).cpu().numpy(), a[:, :, ::-1])


def test_image_batches_larger_than_one_launch(cv, K, orc, gpu):
    # the image-batch operators pack at most a few hundred images' tiles into one launch and loop over
    # the rest: 401 images make every operator issue a second launch, whose images must use their own
    # descriptors, matrices and flip codes
    rng = np.random.default_rng(401)
    n = 401
    bi, hosts = cv.ImageBatchVarShape(n), []
    for i in range(n):
        w, h = int(rng.integers(1, 40)), int(rng.integers(1, 24))
        a = orc.fill_u8((h, w, 3), 9000 + i)
        hosts.append(a)
        bi.push_back(cv.Image.from_numpy(a, K.IMAGE_FORMAT_BGR8))

    def outputs(fmt, size=lambda a: (a.shape[1], a.shape[0])):
        batch, outs = cv.ImageBatchVarShape(n), []
        for a in hosts:
            o = cv.Image.alloc(size(a), fmt)
            outs.append(o)
            batch.push_back(o)
        return batch, outs

    bo, outs = outputs(K.IMAGE_FORMAT_RGB8)
    cv.CvtColor()(None, bi, bo, K.COLOR_BGR2RGB)
    torch.cuda.synchronize()
    for a, o in zip(hosts, outs):
        np.testing.assert_array_equal(o.plane_view(0, np.uint8, 3).cpu().numpy(), a[..., ::-1])

    bo, outs = outputs(K.IMAGE_FORMAT_BGR8)
    codes = rng.integers(-1, 2, n).astype(np.int32)
    cv.Flip(n)(None, bi, bo, cv.Tensor.from_numpy(codes, "N"))
    torch.cuda.synchronize()
    for a, o, code in zip(hosts, outs, codes):
        ref = {1: a[:, ::-1], 0: a[::-1], -1: a[::-1, ::-1]}[int(code)]
        np.testing.assert_array_equal(o.plane_view(0, np.uint8, 3).cpu().numpy(), ref)

    base, scale = np.array([[[[3.0, 5.0, 7.0]]]], np.float32), np.array([[[[0.5, 1.5, 2.0]]]], np.float32)
    for b, s in ((base, scale), (base[..., :1], scale[..., :1])):
        cv.Normalize()(None, bi, cv.Tensor.from_numpy(b, "NHWC"), cv.Tensor.from_numpy(s, "NHWC"), bo, 1.0, 0.0, 0.0, 0)
        torch.cuda.synchronize()
        for a, o in zip(hosts, outs):
            np.testing.assert_array_equal(o.plane_view(0, np.uint8, 3).cpu().numpy(), orc.normalize(a[None], b, s)[0])

    shifts = rng.integers(-3, 4, (n, 2))
    mats = np.array([[1, 0, sx, 0, 1, sy] for sx, sy in shifts], np.float32)
    cv.WarpAffine(n)(None, bi, bo, cv.Tensor.from_numpy(mats, "NW"), NEAREST | 16, 0, (7, 8, 9, 0))  # 16: inverse map
    torch.cuda.synchronize()
    for a, o, m in zip(hosts, outs, mats):
        ref = orc.warp(a[None], a.shape[:2], m, NEAREST, 0, (7, 8, 9, 0), variant=1)[0]
        np.testing.assert_array_equal(o.plane_view(0, np.uint8, 3).cpu().numpy(), ref)

    bg, gouts = outputs(K.IMAGE_FORMAT_U8)
    cv.CvtColor()(None, bi, bg, K.COLOR_BGR2GRAY)
    torch.cuda.synchronize()
    for a, o in zip(hosts, gouts):
        b, g, r = (a[..., k].astype(np.int64) for k in range(3))
        np.testing.assert_array_equal(o.plane_view(0, np.uint8, 1).cpu().numpy()[..., 0],
                                      (b * 3735 + g * 19235 + r * 9798 + (1 << 14)) >> 15)

    for interp in (LINEAR, AREA):
        br, routs = outputs(K.IMAGE_FORMAT_BGR8, lambda a: (a.shape[1] * 2 // 3 + 1, a.shape[0] + 2))
        cv.Resize()(None, bi, br, interp)
        torch.cuda.synchronize()
        for a, o in zip(hosts, routs):
            w, h = o.size
            ref = orc.resize_shipped(a[None], (h, w), interp, varshape=True)[0] if interp == AREA else orc.resize(a[None], (h, w), interp, variant=1)[0]
            got = o.plane_view(0, np.uint8, 3).cpu().numpy()
            assert np.abs(got.astype(np.int32) - ref).max() <= (1 if interp == LINEAR else 0), (interp, a.shape)

    by, youts, yhosts = cv.ImageBatchVarShape(n), [], []
    for i in range(n):
        w, h = 2 * int(rng.integers(1, 20)), 2 * int(rng.integers(1, 12))
        y = np.concatenate([orc.fill_u8((h, w), 100 + i, 16, 235), orc.fill_u8((h // 2, w), 600 + i, 16, 240)])[..., None]
        yhosts.append(y)
        by.push_back(cv.Image.from_numpy(y, K.IMAGE_FORMAT_U8))
        o = cv.Image.alloc((w, h), K.IMAGE_FORMAT_RGB8)
        youts.append(o)
    byo = cv.ImageBatchVarShape(n)
    for o in youts:
        byo.push_back(o)
    cv.CvtColor()(None, by, byo, K.COLOR_YUV2RGB_NV12)
    torch.cuda.synchronize()
    for y, o in zip(yhosts, youts):
        np.testing.assert_array_equal(o.plane_view(0, np.uint8, 3).cpu().numpy()[None],
                                      orc.yuv420_to_rgb(y[None], 3, False, 0, True))


def test_concurrent_submits_on_shared_operator_handles(cv, K, orc, gpu):
    # operators hold no per-call state: several host threads, each with its own stream and tensors,
    # submit through the SAME handles at the same time (ctypes drops the GIL around each call), and
    # create and destroy their tensors concurrently (handle pools). Every thread must get the result a
    # lone thread gets, and an error raised in one thread must not show up in another's status.
    import threading
    resize, swz, norm, fused = cv.Resize(), cv.CvtColor(), cv.Normalize(), cv.ResizeCropConvertReformat()
    b_host, s_host = np.array([[[[3.0, 5.0, 7.0]]]], np.float32), np.array([[[[0.5, 1.5, 2.0]]]], np.float32)
    base, scale = cv.Tensor.from_numpy(b_host, "NHWC"), cv.Tensor.from_numpy(s_host, "NHWC")
    torch.cuda.synchronize()
    n_threads, rounds = 6, 25
    failures, start = [], threading.Barrier(n_threads)

    def worker(tid):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            src = orc.fill_u8((2, 45 + tid, 70 + 3 * tid, 3), 700 + tid)
            want_small = orc.resize_shipped(src, (23, 31), LINEAR)
            want_fused = orc.fused_rccr(src, (16, 16), (32, 24), (5, 3), LINEAR, np.float32, True, 0, 1 / 255.0, 0.0, False)
            start.wait()
            for r in range(rounds):
                with torch.cuda.stream(stream):
                    tin = cv.Tensor.from_numpy(src, "NHWC")
                    t1 = cv.Tensor.alloc([2, 23, 31, 3], np.uint8, "NHWC")
                    t2 = cv.Tensor.alloc([2, 23, 31, 3], np.uint8, "NHWC")
                    t3 = cv.Tensor.alloc([2, 23, 31, 3], np.uint8, "NHWC")
                    t4 = cv.Tensor.alloc([2, 3, 16, 16], np.float32, "NCHW")
                    stream.synchronize()  # the uploads above ran on torch's streams
                    resize(stream, tin, t1, LINEAR)
                    swz(stream, t1, t2, K.COLOR_BGR2RGB)
                    norm(stream, t2, base, scale, t3, 1.0, 0.0, 0.0, 0)
                    fused(stream, tin, t4, (32, 24), LINEAR, (5, 3), 0, 1 / 255.0, 0.0, False)
                    if r % 5 == tid % 5:  # a failing call in this thread only
                        with pytest.raises(cv.Error) as e:
                            resize(stream, tin, t4, LINEAR)
                        assert e.value.status == 2
                    stream.synchronize()
                    got_small, got_norm, got_fused = t1.numpy(), t3.numpy(), t4.numpy()
                assert np.abs(got_small.astype(np.int32) - want_small).max() <= 1
                # the chain's later stages are exact functions of the first stage's output
                np.testing.assert_array_equal(got_norm, orc.normalize(got_small[..., ::-1].copy(), b_host, s_host))
                assert (np.abs(got_fused - want_fused) <= 1e-5 * np.maximum(1.0, np.abs(want_fused))).all()
        except BaseException as exc:  # noqa: BLE001 - reported by the main thread
            failures.append((tid, repr(exc)))
            start.abort()

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not failures, failures


def test_row_pieces_longer_than_one_store_with_odd_lane_counts(cv, K, orc, gpu):
    # 2-byte pixels give 24- or 32-byte pieces per lane, which the run kernels hand round the wave as
    # 16-byte chunks; an odd number of 24-byte pieces ends with half a chunk. Widths chosen so that the
    # number of whole runs per row is 1, 3, 5, 63, 64, 65 (plus a ragged end).
    rng = np.random.default_rng(24)
    for w in (4, 6, 13, 22, 254, 256, 259, 262):
        for c in (3, 4):
            a = rng.integers(0, 65536, (2, 5, w, c)).astype(np.uint16)
            tin = cv.Tensor.from_numpy(a, "NHWC")
            out = cv.Tensor.alloc([2, 5, w, c], np.uint16, "NHWC")
            for code, ref in ((1, a[:, :, ::-1]), (0, a[:, ::-1]), (-1, a[:, ::-1, ::-1])):
                out.torch_view().zero_()
                cv.Flip()(None, tin, out, code)
                torch.cuda.synchronize()
                np.testing.assert_array_equal(out.numpy(), ref, err_msg="flip %d w=%d c=%d" % (code, w, c))
            swapped = cv.Tensor.alloc([2, 5, w, c], np.uint16, "NHWC")
            cv.CvtColor()(None, tin, swapped, K.COLOR_BGR2RGB if c == 3 else K.COLOR_BGRA2RGBA)
            torch.cuda.synchronize()
            want = a.copy()
            want[..., :3] = a[..., 2::-1]
            np.testing.assert_array_equal(swapped.numpy(), want, err_msg="swizzle w=%d c=%d" % (w, c))
        a8 = orc.fill_u8((2, 5, w, 3), 90 + w)
        f = cv.Tensor.alloc([2, 5, w, 3], np.float64, "NHWC")
        cv.ConvertTo()(None, cv.Tensor.from_numpy(a8, "NHWC"), f, 0.5, 1.0)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(f.numpy(), a8.astype(np.float64) * 0.5 + 1.0)


@pytest.mark.parametrize("h,w", [(300000, 16), (16, 300000)])
def test_images_hundreds_of_thousands_of_pixels_tall_or_wide(cv, K, orc, gpu, h, w):
    # launch grids far beyond 65535 blocks in one dimension; every operator in a form whose result is a closed
    # form of the input (identity maps, mirrors, transposes)
    a = orc.fill_u8((1, h, w, 3), 5)
    tin = cv.Tensor.from_numpy(a, "NHWC")

    def run(op, out_shape, dt, layout, *args):
        out = cv.Tensor.alloc(out_shape, dt, layout)
        out.torch_view().fill_(0x5A)
        op(None, tin, out, *args)
        torch.cuda.synchronize()
        return out.numpy()

    same = [1, h, w, 3]
    np.testing.assert_array_equal(run(cv.CvtColor(), same, np.uint8, "NHWC", K.COLOR_BGR2RGB), a[..., ::-1])
    np.testing.assert_array_equal(run(cv.Reformat(), [1, 3, h, w], np.uint8, "NCHW"), a.transpose(0, 3, 1, 2))
    np.testing.assert_array_equal(run(cv.ConvertTo(), same, np.float32, "NHWC", 1.0, 0.0), a.astype(np.float32))
    np.testing.assert_array_equal(run(cv.Flip(), same, np.uint8, "NHWC", 0), a[:, ::-1])
    np.testing.assert_array_equal(run(cv.Flip(), same, np.uint8, "NHWC", 1), a[:, :, ::-1])
    np.testing.assert_array_equal(run(cv.Resize(), same, np.uint8, "NHWC", NEAREST), a)
    np.testing.assert_array_equal(run(cv.Resize(), same, np.uint8, "NHWC", LINEAR), a)
    np.testing.assert_array_equal(run(cv.WarpAffine(0), same, np.uint8, "NHWC", [1, 0, 0, 0, 1, 0], LINEAR, 0, (0, 0, 0, 0)), a)
    np.testing.assert_array_equal(run(cv.CustomCrop(), [1, h - 2, w - 2, 3], np.uint8, "NHWC", (1, 1, w - 2, h - 2)),
                                  a[:, 1:-1, 1:-1])
    zero = cv.Tensor.from_numpy(np.zeros((1, 1, 1, 3), np.float32), "NHWC")
    one = cv.Tensor.from_numpy(np.ones((1, 1, 1, 3), np.float32), "NHWC")
    out = cv.Tensor.alloc(same, np.uint8, "NHWC")
    cv.Normalize()(None, tin, zero, one, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.numpy(), a)
    got = run(cv.ResizeCropConvertReformat(), [1, 3, h, w], np.float32, "NCHW", (w, h), LINEAR, (0, 0), 0, 1.0, 0.0, False)
    np.testing.assert_array_equal(got, a.transpose(0, 3, 1, 2).astype(np.float32))
    gray = run(cv.CvtColor(), [1, h, w, 1], np.uint8, "NHWC", K.COLOR_BGR2GRAY)
    want = (a[..., 0].astype(np.int64) * 3735 + a[..., 1].astype(np.int64) * 19235 + a[..., 2].astype(np.int64) * 9798
            + (1 << 14)) >> 15
    np.testing.assert_array_equal(gray[..., 0], want.astype(np.uint8))
