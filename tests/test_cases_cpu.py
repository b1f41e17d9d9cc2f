"""Host-side checks of the synthetic cases: graph shapes, op counts, and that the oracle evaluation of a
small case produces live (non-degenerate) activations, so that whole-network parity is meaningful."""
import numpy as np

from nart_amd import cases

from oracle import casecpu as case_oracle  # noqa: E402


def test_resnet50_shape_and_ops():
    c = cases.resnet50(N=64)
    convs = [n for n in c.nodes if n.kind == "conv"]
    assert len(convs) == 53 and sum(n.kind == "add" for n in c.nodes) == 16
    assert c.tensors[c.nodes[-2].output].shape == (64, 1000, 1, 1) and c.output.dtype == "f32"
    # 8.18 GOP per image (conv + FC), 523.4 GOP per batch of 64
    assert abs(c.conv_ops() / 64 / 1e9 - 8.18) < 0.02


def test_resnet18_and_mobilenet_shapes():
    c = cases.resnet18(N=1)
    assert sum(n.kind == "conv" for n in c.nodes) == 20 and c.output.shape == (1, 1000, 1, 1)
    m = cases.mobilenet_v2(N=2)
    assert sum(n.kind == "conv" and n.attrs["group"] > 1 for n in m.nodes) == 17
    assert m.output.shape == (2, 1000, 1, 1)


def test_small_case_activations_are_alive():
    c = cases.resnet18(N=1, hw=64)
    vals = case_oracle.run_case(c, case_oracle.random_input(c))
    for node in c.nodes:
        v = vals[node.output]
        assert v.std() > 3.0, (node.kind, node.output, float(v.std()))
        frac_sat = float(((v == 0) | (v == 255)).mean())
        assert frac_sat < 0.75, (node.kind, node.output, frac_sat)


def test_whole_networks_oracle_equals_compiled_reference(ref_ws):
    """Every intermediate tensor of the synthetic networks: oracle == the reference CPU quant module
    (compiled from its own sources), at the real 224x224 geometry for the ResNets."""
    for c in (cases.mobilenet_v2(N=1, hw=96), cases.resnet18(N=1, hw=224), cases.resnet50(N=1, hw=224)):
        x = case_oracle.random_input(c, 1)
        rc = case_oracle.ReferenceCase(c)
        rc.run(x)
        vals = case_oracle.run_case(c, x)
        for n in c.nodes:
            assert np.array_equal(rc.fetch(n.output).view(np.uint8), vals[n.output].view(np.uint8)), (c.name, n.output)
