"""MI355X-native evaluator for the Brokefish network: the registry.

Same shape as the reference registry (brokefish/nn/__init__.py:40-83): every
implementation exposes a class called ``FusedEncoder`` with the same contract, selected
by name.  One implementation lives here, ``"hip"``::

    net = BrokefishNet().eval()
    model = encoder_impl("hip")(net, int8=True)
    policy_logits, promo, value = model.forward_full(boards, control, rep)
    # boards [n, 32] int16, control [n] int16, rep [n] uint8, all on the GPU
    # policy_logits [n, 32, 64] fp16 raw, promo [n, 32, 4] fp16, value [n] fp32
"""
from __future__ import annotations

IMPLEMENTATIONS = ("hip",)

_WHY: dict = {}


def encoder_impl(name: str):
    """The ``FusedEncoder`` class of one implementation; ``ValueError`` for an unknown name."""
    if name == "hip":
        from .hip_impl import FusedEncoder
        return FusedEncoder
    raise ValueError(f"unknown implementation {name!r}, expected one of {IMPLEMENTATIONS}")


def available() -> list:
    """Implementations usable here (library built and a GPU visible), in registry order."""
    found = []
    for name in IMPLEMENTATIONS:
        try:
            encoder_impl(name)
            from . import hip_impl
            hip_impl.load_library()
            import torch
            if not torch.cuda.is_available():
                raise RuntimeError("no GPU visible")
        except Exception as exc:  # noqa: BLE001 - reported through why_unavailable()
            _WHY[name] = f"{type(exc).__name__}: {exc}"
        else:
            found.append(name)
            _WHY.pop(name, None)
    return found


def why_unavailable() -> dict:
    """Why each missing implementation is missing.  Call :func:`available` first."""
    return dict(_WHY)


__all__ = ["IMPLEMENTATIONS", "encoder_impl", "available", "why_unavailable"]
