"""The copy / clone examples of the reference's GPU tests replayed against their expected-output files
(tests/golden/ref/): tensor_copy_01 (zero strides on either side), tensor_copy_02 (scalars through float, double,
complex-double), tensor_copy_05 (zero-stride double source into a float tensor), tensor_copy_09 (a flipped axis:
negative stride), tensor_clone_01 / 02 / 03 (clone keeps the layout, replicate expands zero strides),
tensor_device_cast_01 and tensor_split_01 (slices of a tensor copied to a device). What these scripts ask of the device
module is the strided, converting copy; tensor creation and printing belong to the interface. The examples that name a
second GPU run on one device here. Every case runs on the CPU oracle (always) and on the device library (gpu marker)."""
import numpy as np
import pytest

import helpers as H
import ref_format as RF
from test_ref_fixtures import Engine, load, tensors

ES = {H.FLOAT: 4, H.DOUBLE: 8, H.INT64: 8, H.CDOUBLE: 16}


@pytest.fixture(params=["oracle", pytest.param("device", marks=pytest.mark.gpu)])
def engine(request):
    if request.param == "oracle":
        return Engine(False)
    request.getfixturevalue("hip")
    return Engine(True, request.getfixturevalue("stream"))


def view(parent, shape, strides_elems, offset_elems=0):
    """Ocean tensor of `shape` over a one-dimensional storage array, strides in elements"""
    return np.lib.stride_tricks.as_strided(parent[offset_elems:], shape=shape, strides=[s * parent.itemsize for s in strides_elems], writeable=False)


def dense(shape):
    st, acc = [], 1
    for n in shape:
        st.append(acc); acc *= n
    return st


def test_tensor_copy_01(engine):
    ts = tensors(load("tensor_copy_01"))
    assert len(ts) == 12
    # a = tensor([2,6],[0,0]); b = tensor([2,6],[0,1]); c = tensor([2,2,3],[1,0,0]); d = tensor([2,6],[0,0]), filled with 1, 2, 3, 4
    layouts = [([2, 6], [0, 0], 1), ([2, 6], [0, 1], 6), ([2, 2, 3], [1, 0, 0], 2), ([2, 6], [0, 0], 1)]
    parents = [np.full(n, k + 1, np.float32) for k, (_, _, n) in enumerate(layouts)]
    for k, (shape, strides, _) in enumerate(layouts):
        RF.assert_matches(H.FLOAT, np.array(view(parents[k], shape, strides)), ts[k], "filled tensor %d" % k)
    a = view(parents[0], *layouts[0][:2])
    for k in (1, 2, 3):                                   # b.copy(a); c.copy(a); d.copy(a)
        shape, strides, _ = layouts[k]
        parents[k] = engine.strided_copy(H.FLOAT, H.FLOAT, parents[0], a, parents[k], view(parents[k], shape, strides))
    for k, (shape, strides, _) in enumerate(layouts):
        RF.assert_matches(H.FLOAT, np.array(view(parents[k], shape, strides)), ts[4 + k], "tensor %d after the copies" % k)
        RF.assert_matches(H.FLOAT, parents[k], ts[8 + k], "storage %d after the copies" % k)


def test_tensor_copy_02(engine):
    ts = tensors(load("tensor_copy_02"))
    assert [t.dtype for t in ts] == [H.FLOAT, H.DOUBLE, H.CDOUBLE, H.CDOUBLE, H.CDOUBLE] and all(t.shape == [] for t in ts)
    b = engine.cast(H.INT64, H.FLOAT, np.array([12345], np.int64))            # b.copy(gpu[0](12345))
    RF.assert_matches(H.FLOAT, b.reshape(()), ts[0], "int64 scalar into float")
    b = engine.cast(H.FLOAT, H.DOUBLE, b)
    RF.assert_matches(H.DOUBLE, b.reshape(()), ts[1], "ocean.double(b)")
    b = engine.cast(H.DOUBLE, H.CDOUBLE, b)
    RF.assert_matches(H.CDOUBLE, b.reshape(()), ts[2], "ocean.cdouble(b)")
    RF.assert_matches(H.CDOUBLE, engine.cast(H.INT64, H.CDOUBLE, np.array([54321], np.int64)).reshape(()), ts[3], "b.copy(54321)")
    RF.assert_matches(H.CDOUBLE, engine.cast(H.DOUBLE, H.CDOUBLE, np.array([1.2345])).reshape(()), ts[4], "b.copy(gpu[0](1.2345))")


def test_tensor_copy_05(engine):
    ts = tensors(load("tensor_copy_05"))
    assert len(ts) == 4
    a = np.full(6, 1.0)                                                       # tensor([3,6],[0,1], double, cpu) filled with 1
    b = np.full(18, 2.0, np.float32)                                          # tensor([3,6], float, gpu[0]) filled with 2
    av, bv = view(a, [3, 6], [0, 1]), view(b, [3, 6], [1, 3])
    RF.assert_matches(H.DOUBLE, np.array(av), ts[0], "a"); RF.assert_matches(H.FLOAT, np.array(bv), ts[1], "b")
    b = engine.strided_copy(H.DOUBLE, H.FLOAT, a, av, b, bv)
    RF.assert_matches(H.DOUBLE, np.array(av), ts[2], "a afterwards"); RF.assert_matches(H.FLOAT, np.array(view(b, [3, 6], [1, 3])), ts[3], "b.copy(a)")


def test_tensor_copy_09(engine):
    ts = tensors(load("tensor_copy_09"))
    assert len(ts) == 4
    a = RF.to_storage(H.FLOAT, ts[0].values).ravel(order="F").copy()          # 4 x 3, values 0..11
    b = RF.to_storage(H.FLOAT, ts[1].values).ravel(order="F").copy()          # 4 x 3, values 12..23
    flipped = np.lib.stride_tricks.as_strided(b[8:], shape=[4, 3], strides=[4, -16], writeable=False)    # b.flipAxis(1, True): a view
    RF.assert_matches(H.FLOAT, np.array(flipped), ts[2], "b.flipAxis(1, True)")
    a = engine.strided_copy(H.FLOAT, H.FLOAT, b, flipped, a, view(a, [4, 3], [1, 4]))                    # a.copy(b)
    got = np.array(np.lib.stride_tricks.as_strided(a[3:], shape=[4, 3], strides=[-4, 16], writeable=False))   # a.flipAxis(0)
    RF.assert_matches(H.FLOAT, got, ts[3], "a.copy(b); a.flipAxis(0)")


def test_tensor_clone_01_03_device_cast_01(engine):
    for name, dtypes in (("tensor_clone_01", [H.FLOAT, H.FLOAT, H.DOUBLE, H.DOUBLE]), ("tensor_clone_03", [H.INT64, H.INT64]),
                         ("tensor_device_cast_01", [H.INT64, H.INT64, H.DOUBLE])):
        ts = tensors(load(name))
        assert [t.dtype for t in ts] == dtypes
        for k, t in enumerate(ts):                       # every printed tensor is a copy of the first of its type onto another device
            src = next(u for u in ts if u.dtype == t.dtype and u.shape == t.shape)
            x = RF.to_storage(t.dtype, src.values)
            RF.assert_matches(t.dtype, engine.cast(t.dtype, t.dtype, x), t, "%s item %d" % (name, k))


def test_tensor_clone_02(engine):
    items = load("tensor_clone_02")
    ts = tensors(items)
    assert len(ts) == 4 and [i for i in items if i == ("text", "(4, 8)")]
    store = np.array([1, 2, 3], np.float32)               # t = tensor([2,3],[0,1], float); t.copy([[1,2,3]])
    t = view(store, [2, 3], [0, 1])
    RF.assert_matches(H.FLOAT, np.array(t), ts[0], "t"); RF.assert_matches(H.FLOAT, store, ts[1], "t.storage")
    # clone keeps strides (0, 4): the storage of three elements is copied as it is
    RF.assert_matches(H.FLOAT, engine.cast(H.FLOAT, H.FLOAT, store.reshape(3, 1)).ravel(), ts[2], "t.clone(gpu[0]).storage")
    # replicate expands the zero stride: a dense 2 x 3 tensor with strides (4, 8)
    target = np.zeros(6, np.float32)
    rep = engine.strided_copy(H.FLOAT, H.FLOAT, store, t, target, view(target, [2, 3], [1, 2]))
    RF.assert_matches(H.FLOAT, rep, ts[3], "t.replicate(gpu[0]).storage")


def test_tensor_split_01(engine):
    ts = tensors(load("tensor_split_01"))
    a = RF.to_storage(H.FLOAT, ts[0].values).ravel(order="F").copy()          # 5 x 6, values 0..29
    assert ts[0].shape == [5, 6] and len(ts) == 9
    def piece(axis, start, count):
        shape = [5, 6]; shape[axis] = count
        src = view(a, shape, [1, 5], start * (1 if axis == 0 else 5))
        if count == 0:
            return np.zeros(shape, np.float32)
        target = np.zeros(shape[0] * shape[1], np.float32)
        out = engine.strided_copy(H.FLOAT, H.FLOAT, a, src, target, view(target, shape, dense(shape)))
        return out.reshape(shape, order="F")
    # a.split(0, [cpu, gpu[0], cpu]): rows 0-1, 2-3, 4;  a.split(1, [1, 5, 0]);  a.split(0, [gpu[0], cpu], [1, 4])
    expect = [(0, 0, 2), (0, 2, 2), (0, 4, 1), (1, 0, 1), (1, 1, 5), (1, 6, 0), (0, 0, 1), (0, 1, 4)]
    for k, (axis, start, count) in enumerate(expect):
        want = ts[1 + k]
        shape = [5, 6]; shape[axis] = count
        assert want.shape == shape, (k, want.shape)
        if count:
            RF.assert_matches(H.FLOAT, piece(axis, start, count), want, "split piece %d" % k)
