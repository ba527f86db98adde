"""The TorchScript custom classes (lib/libcuda_mace.so): registration, method schemas and pickling, checked without a GPU."""
import io

import pytest
import torch


@pytest.fixture(scope="module")
def classes():
    from cuda_mace.ops import classes as C

    return C


EXPECTED = {
    ("inv_message_passing", "InvariantMessagePassingTP"): ["X", "Y", "raidal", "sender_list", "receiver_list", "nnodes"],
    ("spherical_harmonics", "SphericalHarmonics"): ["xyz"],
    ("cubic_spline", "CubicSpline"): ["r", "r_knots", "coeffs", "r_width", "r_max"],
    ("linear_wmma", "Linear"): ["X", "W", "W_T"],
    ("linear_wmma", "ElementalLinear"): ["X", "W", "W_T", "one_hot_encoding"],
    ("symm_contract", "SymmetricContraction"): [
        "X", "atom_types", "U3_max_nonsparse", "U3_num_nonzero", "U3_indices", "U3_values", "U2_num_nonzero", "U2_indices",
        "U2_values", "U1_num_nonzero", "U1_index", "W3", "W2", "W1", "W3_size", "W2_size", "W1_size"],
}


@pytest.mark.parametrize("key", sorted(EXPECTED), ids=lambda k: ".".join(k))
def test_class_is_registered_with_the_reference_schema(classes, key):
    ns, name = key
    obj = getattr(getattr(torch.classes, ns), name)()
    schema = obj._get_method("forward").schema
    args = [a.name for a in schema.arguments][1:]  # drop self
    assert args == EXPECTED[key]
    assert str(schema.returns[0].type) == "Tensor"


class Holder(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.cuda_obj = torch.classes.linear_wmma.Linear()
        self.register_buffer("w", torch.ones(3))


def test_objects_pickle_with_empty_state(classes):
    buf = io.BytesIO()
    torch.save(Holder(), buf)
    buf.seek(0)
    back = torch.load(buf, weights_only=False)
    assert isinstance(back.cuda_obj, torch.ScriptObject) and torch.equal(back.w, torch.ones(3))


def test_host_tensors_are_rejected(classes):
    with pytest.raises(RuntimeError, match="GPU"):
        torch.classes.spherical_harmonics.SphericalHarmonics().forward(torch.zeros(4, 3))
    with pytest.raises(RuntimeError, match="GPU"):
        torch.classes.linear_wmma.Linear().forward(torch.zeros(2, 16, 32), torch.zeros(4, 32, 32), torch.zeros(4, 32, 32))
