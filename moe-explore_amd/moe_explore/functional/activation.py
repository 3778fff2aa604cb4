"""Activation names and their plain-PyTorch definitions.

Mirrors the reference's ``functional/activation.py:5-26``: four public names,
and the GLU variants read an *interleaved* layout, gate = even columns,
up = odd columns (``functional/activation.py:19-20``).
"""
import enum

import torch


class Activation(str, enum.Enum):
    # A str-valued enum, so that ``"glu" in params.activation`` and dict lookups
    # keyed by the plain string both work, as with the reference's StrEnum.
    SILU = "silu"
    GELU = "gelu"
    SWIGLU = "swiglu"
    GEGLU = "geglu"

    def __str__(self):
        return self.value


_NAMES = {a.value for a in Activation}


def activation_name(act):
    """Plain string for an activation given as None, str or Activation."""
    if act is None:
        return None
    return act.value if isinstance(act, Activation) else str(act)


def is_glu(act):
    name = activation_name(act)
    return name is not None and "glu" in name


def glu_form(act):
    """Activation of a gated record (``GLUParams`` / ``GLUInterleavedParams``, ``params.py:16-27``)
    given as the model's ``hidden_act``: "silu" means SwiGLU and "gelu" GeGLU, the rule of the
    reference's ``tests/test_hf.py:61-64``; GLU names pass through."""
    name = activation_name(act)
    if name is None or is_glu(name):
        return act
    return "geglu" if name == "gelu" else "swiglu"


def activation(x: torch.Tensor, activation: "Activation | str"):
    name = activation_name(activation)
    assert name in _NAMES, f"Invalid activation: {activation}"
    if name == "silu":
        return torch.nn.functional.silu(x)
    if name == "gelu":
        return torch.nn.functional.gelu(x)
    assert x.shape[-1] % 2 == 0
    gate = x[..., 0::2]
    up = x[..., 1::2]
    if name == "swiglu":
        gate = torch.nn.functional.silu(gate)
    else:
        gate = torch.nn.functional.gelu(gate)
    return gate * up
