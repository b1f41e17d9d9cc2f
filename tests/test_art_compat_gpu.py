"""The reference's Python usage (python/nart/art/__init__.py:20-27), run unchanged against nart_amd.art_compat: an
engine file and its JSON configuration on disk, create_context_from_json / load_parade / get_empty_io / Parade.run,
the output compared with the CPU oracle bit for bit."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from nart_amd import art_compat as art  # noqa: E402  (the one line a NART user changes)
from nart_amd import cases, engine  # noqa: E402
from oracle import casecpu  # noqa: E402  (checker only)


def _write(tmp_path, case):
    fp = os.path.join(tmp_path, case.name + ".bin")
    with open(fp, "wb") as f:
        f.write(engine.write_engine(case))
    with open(fp + ".json", "w") as f:
        json.dump({"workspaces": {"hip": {}}, "input_workspace": "hip"}, f)
    return fp


def test_readme_usage_on_resnet18(tmp_path):
    case = cases.resnet18(N=2, hw=96)
    fp = _write(str(tmp_path), case)
    rng = np.random.default_rng(5)
    x = rng.integers(0, 256, case.input.shape, dtype=np.uint8)
    want = casecpu.run_case(case, x)[case.output.name].reshape(2, -1)  # the runtime infers [N, K] for an inner product (art/src/op.c)

    ctx = art.create_context_from_json(fp + ".json")
    assert ctx.loaded_workspaces == ["hip"]
    parade = art.load_parade(fp, ctx)
    inputs, outputs = art.get_empty_io(parade)
    assert list(inputs) == [case.input.name] and list(outputs) == [case.output.name]
    inputs[case.input.name][:] = x
    assert parade.run(inputs, outputs) is True
    got = outputs[case.output.name]
    assert got.dtype == want.dtype and got.shape == want.shape and np.array_equal(got, want)

    # the rest of the surface (module.cpp:302-400)
    assert parade.input_shapes() == {case.input.name: list(case.input.shape)}
    assert parade.output_shapes() == {case.output.name: list(want.shape)}
    assert parade.input_dtypes() == {case.input.name: "uint8"} and parade.output_dtypes() == {case.output.name: str(want.dtype)}
    assert parade.get_tensor_dtype(case.input.name) == "uint8" and parade.get_tensor_dtype("no such tensor") is None
    assert parade.get_tensor_shape(case.output.name) == list(want.shape) and parade.get_tensor_shape("nope") is None
    assert parade.get_input_names() == [case.input.name] and parade.get_output_names() == [case.output.name]
    assert parade.get_raw_tensor_data(case.input.name) != 0 and parade.get_raw_tensor_data("nope") == 0

    # wrong arguments raise what the reference raises
    with pytest.raises(ValueError, match="input shape not match"):
        parade.run({case.input.name: x[:1]}, outputs)
    with pytest.raises(ValueError, match="input dtype not match"):
        parade.run({case.input.name: x.astype(np.float32)}, outputs)
    with pytest.raises(ValueError, match="input dim size not match"):
        parade.run({case.input.name: x.reshape(-1)}, outputs)
    with pytest.raises(ValueError, match="output dtype not match"):
        parade.run(inputs, {case.output.name: got.astype(np.float64)})

    # reshape to another batch (module.cpp:381-400), then run again
    shape = list(case.input.shape)
    shape[0] = 3
    assert parade.reshape({case.input.name: shape}) is True
    assert parade.reshape({case.input.name: shape[:3]}) is False  # rank mismatch
    inputs3, outputs3 = art.get_empty_io(parade)
    x3 = rng.integers(0, 256, shape, dtype=np.uint8)
    inputs3[case.input.name][:] = x3
    parade.run(inputs3, outputs3)
    want3 = casecpu.run_case(cases.resnet18(N=3, hw=96), x3)[case.output.name].reshape(3, -1)
    assert np.array_equal(outputs3[case.output.name], want3)
    # forward() alone re-runs on what the input memory holds
    parade.forward()


def test_float_network_ends_and_missing_modules(tmp_path):
    case = cases.resnet50(N=1, hw=64)  # fp32 input -> quantize ... dequantize -> fp32 output
    fp = _write(str(tmp_path), case)
    rng = np.random.default_rng(6)
    x = (rng.standard_normal(case.input.shape) * 1.2).astype(np.float32)
    want = casecpu.run_case(case, x)[case.output.name].reshape(1, -1)
    # a module that does not exist is skipped with a message, like the reference (module.cpp:104-110)
    ctx = art.RuntimeContext(["no_such_module", "hip"], "hip")
    assert ctx.loaded_workspaces == ["hip"]
    parade = art.load_parade(fp, ctx)
    inputs, outputs = art.get_empty_io(parade)
    assert inputs[case.input.name].dtype == np.float32
    inputs[case.input.name][:] = x
    parade.run(inputs, outputs)
    assert np.array_equal(outputs[case.output.name].view(np.uint32), want.view(np.uint32))
    ctx2 = art.create_context_for_target("hip")
    assert ctx2.loaded_workspaces == ["hip"]
