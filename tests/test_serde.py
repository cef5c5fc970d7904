"""The tensor wire format of the reference (src/tensor.rs:1199-1249), pinned by its own token test
(src/tensor.rs:2236-2277), and the layer structs' data model around it (layer.rs:833-848, 1069-1073, 1150-1155:
field lists of the derive; no vector of them exists in the reference).  CPU only but for the device round trips: the
encoding is host logic."""
import json

import numpy as np
import pytest

from autograph_amd import serde


def test_token_stream_matches_the_reference_test_vector():
    # tensor_serde: data = [1u32, 2, 3, 4]; the items are the bytes taken 8 at a time, big-endian
    data = np.array([1, 2, 3, 4], dtype=np.uint32)
    items = [int.from_bytes(data[:2].tobytes(), "big"), int.from_bytes(data[2:].tobytes(), "big")]
    assert items == [0x0100000002000000, 0x0300000004000000]  # = u64::to_be of the native-endian pairs
    want = [("Struct", "Tensor", 2), ("Str", "dim"), ("Tuple", 1), ("U64", 4), ("TupleEnd",), ("Str", "buffer"),
            ("TupleStruct", "Buffer", 3), ("Str", "U32"), ("U64", 4), ("Seq", 2), ("U64", items[0]), ("U64", items[1]),
            ("SeqEnd",), ("TupleStructEnd",), ("StructEnd",)]
    assert serde.to_tokens(data) == want


def test_json_is_the_same_data_model():
    data = np.array([1, 2, 3, 4], dtype=np.uint32)
    text = serde.to_json(data)
    assert text == '{"dim":[4],"buffer":["U32",4,[72057594071482368,216172782180892672]]}'
    back, is_bf16 = serde.from_json(text)
    assert not is_bf16 and back.dtype == np.uint32 and np.array_equal(back, data)


@pytest.mark.parametrize("shape", [(1,), (3,), (2, 3), (6, 1, 5, 5), (84, 10), (0, 4)])
@pytest.mark.parametrize("kind", ["f32", "bf16"])
def test_round_trip(shape, kind):
    rng = np.random.default_rng(3)
    if kind == "f32":
        a = rng.standard_normal(shape).astype(np.float32)
    else:
        a = rng.integers(0, 1 << 16, shape).astype(np.uint16)
    text = serde.to_json(a, bf16=kind == "bf16")
    obj = json.loads(text)
    assert obj["dim"] == list(shape) and obj["buffer"][0] == ("F32" if kind == "f32" else "BF16")
    assert obj["buffer"][1] == a.size and len(obj["buffer"][2]) == -(-a.nbytes // 8)
    back, is_bf16 = serde.from_json(text)
    assert is_bf16 == (kind == "bf16") and back.shape == tuple(shape) and np.array_equal(back, a)
    # the token stream carries the same items
    toks = serde.to_tokens(a, bf16=kind == "bf16")
    assert [t[1] for t in toks if t[0] == "U64"][a.ndim + 1:] == obj["buffer"][2]


def test_rejects_what_the_reference_rejects():
    good = json.loads(serde.to_json(np.arange(6, dtype=np.float32).reshape(2, 3)))
    for mutate in (lambda o: o.pop("dim"), lambda o: o.update(extra=1), lambda o: o.__setitem__("dim", [4, 2]),
                   lambda o: o["buffer"].__setitem__(0, "F31"), lambda o: o["buffer"][2].append(0),
                   lambda o: o["buffer"].__setitem__(1, 7), lambda o: o["buffer"][2].__setitem__(0, -1),
                   lambda o: o["buffer"][2].__setitem__(0, 1 << 64)):
        o = json.loads(json.dumps(good))
        mutate(o)
        with pytest.raises(serde.SerdeError):
            serde.from_json(json.dumps(o))
    with pytest.raises(serde.SerdeError):
        serde.from_json("[1, 2")


@pytest.mark.gpu
def test_device_tensor_round_trip():
    import autograph_amd as ag
    import oracle as orc
    ag.Device(0)
    rng = np.random.default_rng(4)
    w = rng.standard_normal((16, 6, 5, 5)).astype(np.float32)
    for arr, dt in ((w, "f32"), (orc.f32_to_bf16(w), "bf16")):
        t = ag.Tensor.from_array(arr)
        back = ag.Tensor.from_json(t.to_json(), dtype=dt)
        assert back.dtype == dt and np.array_equal(back.into_array(), arr)
        # a transposed view is written in standard layout
        v = ag.Tensor.from_array(arr.reshape(16, 150)).t()
        assert np.array_equal(ag.Tensor.from_json(v.to_json()).into_array(), arr.reshape(16, 150).T)
    with pytest.raises(ag.AghError):
        ag.Tensor.from_json(ag.Tensor.from_array(w).to_json(), dtype="bf16")
    with pytest.raises(ag.AghError):
        ag.Tensor.from_json(serde.to_json(np.arange(4, dtype=np.uint32)))


def test_layer_values_follow_the_derived_field_lists():
    rng = np.random.default_rng(5)
    w = rng.standard_normal((4, 3, 5, 5)).astype(np.float32)
    b = rng.standard_normal(4).astype(np.float32)
    v = serde.conv2_to_value(w, b, padding=(2, 1), stride=(1, 2), dilation=(1, 1))
    assert list(v) == ["weight", "padding", "stride", "dilation", "bias"]          # layer.rs:842-848
    assert list(v["weight"]) == ["value"] and v["weight"]["value"] == json.loads(serde.to_json(w))
    assert v["padding"] == [2, 1] and v["stride"] == [1, 2] and v["dilation"] == [1, 1]
    back = serde.conv2_from_value(json.loads(json.dumps(v)))
    assert np.array_equal(back["weight"][0], w) and np.array_equal(back["bias"][0], b) and not back["weight"][1]
    assert (back["padding"], back["stride"], back["dilation"]) == ((2, 1), (1, 2), (1, 1))
    assert serde.conv2_from_value(serde.conv2_to_value(w))["bias"] is None            # Option::None is null
    d = serde.dense_to_value(w.reshape(4, 75), None)
    assert list(d) == ["weight", "bias"] and d["bias"] is None                        # layer.rs:1070-1073
    assert np.array_equal(serde.dense_from_value(d)["weight"][0], w.reshape(4, 75))
    assert serde.max_pool2_to_value((2, 2), (2, 2)) == {"filter": [2, 2], "stride": [2, 2]}  # layer.rs:1152-1155
    assert serde.max_pool2_from_value({"filter": [3, 2], "stride": [1, 1]}) == dict(filter=(3, 2), stride=(1, 1))
    # an absent optimizer state is the default (none); a null one is no state (the deserializer reads a struct,
    # autograd.rs:1141-1151); missing non-optional fields and wrong ranks are errors
    assert serde.parameter_from_value({"value": json.loads(serde.to_json(b))}, 1).optim_state is None
    with pytest.raises(serde.SerdeError):
        serde.parameter_from_value({"value": json.loads(serde.to_json(b)), "optim_state": None}, 1)
    for bad in ({"bias": None}, {"weight": {"value": json.loads(serde.to_json(b))}, "bias": None}):
        with pytest.raises(serde.SerdeError):
            serde.dense_from_value(bad)
    # the derives set no `deny_unknown_fields` (layer.rs:833-848, :1069-1073, autograd.rs:639-656): a key they do not
    # know is skipped and a missing `Option` field is None, at every level
    lenient = serde.dense_from_value({"weight": {**d["weight"], "note": 1}, "extra": [1, 2]})
    assert lenient["bias"] is None and np.array_equal(lenient["weight"][0], w.reshape(4, 75))
    cv = {k: val for k, val in v.items() if k != "bias"}
    assert serde.conv2_from_value({**cv, "future_field": None})["bias"] is None
    assert serde.max_pool2_from_value({"filter": [2, 2], "stride": [2, 2], "x": 0}) == dict(filter=(2, 2), stride=(2, 2))
    with pytest.raises(serde.SerdeError):
        serde.conv2_from_value({k: val for k, val in v.items() if k != "stride"})
    with pytest.raises(serde.SerdeError):
        serde.conv2_from_value({**v, "padding": [1]})
    with pytest.raises(serde.SerdeError):
        serde.max_pool2_from_value({"filter": [2, 2]})


def test_parameter_optimizer_state_follows_the_derived_field_lists():
    """`optim_state` after `value`, only when there is a state (autograd.rs:647-656); a state is its name and its
    (key, value) pairs, the optimizer's type id skipped (optimizer.rs:166-173); a value is the externally tagged
    `Tensor` variant with the tensor and the two flags SGD sets (optimizer.rs:108-131, :373-380)."""
    rng = np.random.default_rng(8)
    w = rng.standard_normal((3, 4)).astype(np.float32)
    vel = rng.standard_normal((3, 4)).astype(np.float32)
    state = serde.OptimStateValue("SGD", [("velocity", vel, False, True, True)])
    v = serde.parameter_to_value(w, optim_state=state)
    assert list(v) == ["value", "optim_state"] and list(v["optim_state"]) == ["name", "key_values"]
    assert v["optim_state"]["name"] == "SGD"
    (key, value), = v["optim_state"]["key_values"]
    assert key == "velocity" and list(value) == ["Tensor"]
    assert list(value["Tensor"]) == ["tensor", "parameter_device", "parameter_type"]
    assert value["Tensor"]["tensor"] == json.loads(serde.to_json(vel))
    assert value["Tensor"]["parameter_device"] is True and value["Tensor"]["parameter_type"] is True
    back = serde.parameter_from_value(json.loads(json.dumps(v)), 2)
    assert np.array_equal(back[0], w) and back.optim_state.name == "SGD"
    (k, a, is_bf16, pdev, ptype), = back.optim_state.key_values
    assert k == "velocity" and np.array_equal(a, vel) and not is_bf16 and pdev and ptype
    # SGD without momentum: a state with no values (optimizer.rs:366-381)
    empty = serde.parameter_to_value(w, optim_state=serde.OptimStateValue("SGD"))
    assert empty["optim_state"] == {"name": "SGD", "key_values": []}
    assert serde.parameter_from_value(empty, 2).optim_state.key_values == []
    # bf16 velocity, inside a layer
    bits = (vel.view(np.uint32) >> 16).astype(np.uint16)
    d = serde.dense_to_value(bits, None, bf16=True, weight_state=serde.OptimStateValue("SGD", [("velocity", bits, True, True, True)]))
    got = serde.dense_from_value(json.loads(json.dumps(d)))["weight"]
    assert got[1] and got.optim_state.key_values[0][2] and np.array_equal(got.optim_state.key_values[0][1], bits)
    for bad in ({"name": "SGD"}, {"name": "SGD", "key_values": [["velocity", {"Elem": {"F32": 0.5}}]]},
                {"name": "SGD", "key_values": [["velocity", {"Tensor": {"tensor": value["Tensor"]["tensor"]}}]]},
                {"name": "SGD", "key_values": [["velocity"]]}, {"name": 3, "key_values": []}):
        with pytest.raises(serde.SerdeError):
            serde.parameter_from_value({"value": v["value"], "optim_state": bad}, 2)


@pytest.mark.gpu
def test_trainer_velocity_is_written_with_the_parameters():
    """A LeNet5 training step with momentum, then every layer written and read back: the velocity travels as the
    parameter's optimizer state and is the trainer's, bit for bit; a layer without a trainer writes none."""
    import autograph_amd as ag
    ag.Device(0)
    rng = np.random.default_rng(12)

    def he(shape, fan_in):
        a = np.sqrt(2.0 / fan_in)
        return rng.uniform(-a, a, shape).astype(np.float32)

    def lenet():
        return ag.LeNet5.from_arrays(he((6, 1, 5, 5), 25), he((16, 6, 5, 5), 150), he((256, 128), 256), he((128, 84), 128),
                                     he((84, 10), 84), he((10,), 84))

    model = lenet()
    assert "optim_state" not in json.loads(model.dense1.to_json())["weight"]
    trainer = ag.LeNet5Trainer(model, 16, learning_rate=0.05, optimizer=ag.SGD(momentum=0.9))
    x = ag.Tensor.from_array(rng.uniform(0, 1, (16, 1, 28, 28)).astype(np.float32))
    labels = rng.integers(0, 10, 16).astype(np.uint8)
    t = ag.Buffer(labels.size)
    ag._ffi.check(ag.lib.agh_memcpy_h2d(t.ptr, labels.ctypes.data, labels.size))
    ag._ffi.check(ag.lib.agh_sync())
    trainer.step(x, t)
    trainer.step(x, t)
    ag._ffi.check(ag.lib.agh_sync())
    for layer, vel in ((model.conv1, trainer.velocities[0]), (model.dense1, trainer.velocities[2]), (model.dense3, trainer.velocities[4])):
        back = type(layer).from_json(layer.to_json())
        assert back.weight_state.name == "SGD"
        v = back.weight_state.get("velocity").into_array()
        assert np.array_equal(v, vel.into_array()) and np.abs(v).max() > 0
        assert np.array_equal(back.weight.into_array(), layer.weight.into_array())
        # written again, the state is still there
        assert json.loads(back.to_json())["weight"]["optim_state"]["name"] == "SGD"
    back = ag.Dense.from_json(model.dense3.to_json())
    assert np.array_equal(back.bias_state.get("velocity").into_array(), trainer.velocities[5].into_array())
    plain = ag.LeNet5Trainer(lenet(), 16)
    assert json.loads(plain.model.dense2.to_json())["weight"]["optim_state"] == {"name": "SGD", "key_values": []}


@pytest.mark.gpu
def test_device_layer_round_trip():
    import autograph_amd as ag
    import oracle as orc
    ag.Device(0)
    rng = np.random.default_rng(6)
    w = rng.standard_normal((6, 1, 5, 5)).astype(np.float32)
    b = rng.standard_normal(6).astype(np.float32)
    x = rng.standard_normal((2, 1, 12, 12)).astype(np.float32)
    for dt, conv in (("f32", lambda a: a), ("bf16", orc.f32_to_bf16)):
        layer = ag.Conv2(ag.Tensor.from_array(conv(w)), ag.Tensor.from_array(conv(b)), padding=(1, 1))
        back = ag.Conv2.from_json(layer.to_json(), dtype=dt)
        assert back.padding == (1, 1) and back.stride == (1, 1) and back.weight.dtype == dt
        tx = ag.Tensor.from_array(conv(x))
        assert np.array_equal(back.forward(tx).into_array(), layer.forward(tx).into_array())
        dense = ag.Dense(ag.Tensor.from_array(conv(w.reshape(6, 25).T.copy())))
        back = ag.Dense.from_json(dense.to_json())
        assert back.bias is None and np.array_equal(back.weight.into_array(), dense.weight.into_array())
        with pytest.raises(ag.AghError):
            ag.Conv2.from_json(layer.to_json(), dtype="f32" if dt == "bf16" else "bf16")
    pool = ag.MaxPool2.from_json(ag.MaxPool2((2, 2)).to_json())
    assert pool.filter == (2, 2) and pool.stride == (2, 2)
