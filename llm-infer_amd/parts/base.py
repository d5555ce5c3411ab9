"""The interface of a part.

A part is built from the parameters of its ``PartSpec`` plus ``prefix`` (of its
tensor names), ``dtype`` (the compute dtype) and ``device``.  It states the tensors
it needs under local names (``params``), is handed them once (``bind``), and then
runs on the tokens of a step.  Activations between parts: the residual stream is
float32 ``[T, hidden]``; a norm turns it into the compute dtype; a mixer or a
feed-forward adds its result into the residual stream in place.
"""
from __future__ import annotations


class Part:
    prefix: str = ""
    # False for a part whose forward pass waits for the device (a data-dependent shape, a copy to
    # the host): such a step cannot be recorded, and decoding then runs it eagerly.
    recordable: bool = True

    def params(self) -> dict:
        """local tensor name -> ParamSpec"""
        return {}

    def bind(self, tensors: dict) -> None:
        """Receives the tensors of ``params()`` under their local names, on the device."""

    def children(self) -> list:
        return []

    def ignorable(self) -> list:
        """Full tensor names that a checkpoint may hold without this model using them."""
        return []


def collect_params(part: Part, out: dict | None = None) -> dict:
    """Full tensor name -> (owning part, local name, ParamSpec) for a part and all below it."""
    out = {} if out is None else out
    for local, spec in part.params().items():
        name = part.prefix + local
        if name in out:
            raise ValueError(f"two parts claim the tensor {name}")
        out[name] = (part, local, spec)
    for c in part.children():
        collect_params(c, out)
    return out
