"""Host-side operator API (the mirror of ma/monarch_attention.py) - no GPU."""
import pytest
import torch

from ma import monarch_attention as api
from ma.ma_hip import monarch_attention_hip
from ma.monarch_attention import MonarchAttention, PadType, register_impl


def test_pad_type_behaves_like_a_string_enum():
    assert PadType.pre == "pre" and PadType.post == "post"
    assert PadType("pre") is PadType.pre
    assert str(PadType.post) == "post" and f"{PadType.pre}" == "pre"
    assert [p.value for p in PadType] == ["pre", "post"]


def test_unknown_impl_raises_reference_message():
    with pytest.raises(ValueError, match=r"Unknown impl 'nope'\. Available: .*hip"):
        MonarchAttention(16, 2, PadType.pre, impl="nope")


def test_module_is_stateless_and_keeps_its_knobs():
    m = MonarchAttention(14, 3, "pre")
    assert (m.block_size, m.num_steps, m.pad_type) == (14, 3, "pre")
    assert len(list(m.parameters())) == 0 and len(m.state_dict()) == 0
    assert m._impl_fn is monarch_attention_hip


def test_register_impl_and_argument_marshalling():
    seen = {}

    def fake(q, k, v, mask, T, B, pre_pad):
        seen.update(q=q, k=k, v=v, mask=mask, T=T, B=B, pre_pad=pre_pad)
        return v

    register_impl("fake", fake)
    try:
        q, k, v = torch.zeros(1, 1, 6, 4), torch.ones(1, 1, 6, 4), torch.full((1, 1, 6, 4), 2.0)
        for pad, flag in ((PadType.pre, True), ("pre", True), (PadType.post, False), ("post", False)):
            out = MonarchAttention(3, 2, pad, impl="fake")(q, k, v)
            assert out is v and seen["pre_pad"] is flag and seen["mask"] is None
            assert (seen["T"], seen["B"]) == (2, 3) and seen["q"] is q and seen["k"] is k
        mask = torch.ones(1, 6, dtype=torch.bool)
        MonarchAttention(3, 1, "post", impl="fake")(q, k, v, mask)
        assert seen["mask"] is mask
        # get_matrix applies the forward pass to an fp32 identity (reference :61-66)
        MonarchAttention(3, 1, "post", impl="fake").get_matrix(q.half(), k.half())
        assert seen["v"].shape == (1, 1, 6, 6) and seen["v"].dtype == torch.float32
        assert torch.equal(seen["v"][0, 0], torch.eye(6))
    finally:
        api._IMPLEMENTATIONS.pop("fake")


def test_get_matrix_takes_the_identity_route_when_the_matrix_kernel_declines(monkeypatch):
    calls = []

    def decline(*args, **kwargs):
        calls.append(args)
        raise NotImplementedError("padded sequence too long")

    monkeypatch.setattr(api, "monarch_matrix_hip", decline)
    q, k = torch.zeros(1, 1, 6, 4), torch.ones(1, 1, 6, 4)
    # CPU tensors: the forward pass of "hip" refuses them, which shows that it was reached
    with pytest.raises(ValueError, match="GPU"):
        MonarchAttention(3, 1, "pre").get_matrix(q, k)
    assert len(calls) == 1 and calls[0][3:] == (1, 3, True)


def _qkv(dtype=torch.float16):
    return (torch.randn(1, 2, 8, 4, dtype=dtype) for _ in range(3))


def test_hip_impl_refuses_cpu_tensors_instead_of_falling_back():
    q, k, v = _qkv()
    with pytest.raises(ValueError, match="GPU"):
        monarch_attention_hip(q, k, v, None, 1, 4, False)


@pytest.mark.parametrize("mutate,exc", [
    (lambda a: a.update(k=a["k"][:, :, :4]), ValueError),
    (lambda a: a.update(v=a["v"][:, :1]), ValueError),
    (lambda a: a.update(k=a["k"].float()), TypeError),
    (lambda a: a.update(q=a["q"].double(), k=a["k"].double()), TypeError),
    (lambda a: a.update(q=a["q"][0]), ValueError),
    (lambda a: a.update(B=0), ValueError),
    (lambda a: a.update(T=0), ValueError),
    (lambda a: a.update(mask=torch.ones(1, 7)), ValueError),
])
def test_argument_validation(mutate, exc):
    q, k, v = _qkv()
    a = dict(q=q, k=k, v=v, mask=None, T=2, B=4)
    mutate(a)
    with pytest.raises(exc):
        monarch_attention_hip(a["q"], a["k"], a["v"], a["mask"], a["T"], a["B"], False)
