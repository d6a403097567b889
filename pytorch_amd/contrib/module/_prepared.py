"""Bookkeeping for the optional prepared (re-laid-out) weight copies of the quantized linear layers."""
from __future__ import annotations


class PreparedCopiesMixin:
    """A module's ``prepare_()`` keeps derived copies of its parameters in plain attributes.  Anything that moves,
    casts or reloads the parameters (``.to()``, ``.cuda()``, ``.half()``, ``load_state_dict``) would leave those copies
    stale or on the wrong device, so every such operation drops them; the next forward pass then runs on the
    parameters themselves until ``prepare_()`` is called again."""

    _prepared_attrs: tuple = ()

    def _drop_prepared(self) -> None:
        for name in self._prepared_attrs:
            if self.__dict__.get(name) is not None:
                self.__dict__[name] = None

    def _apply(self, fn, *args, **kwargs):
        self._drop_prepared()
        return super()._apply(fn, *args, **kwargs)

    def _load_from_state_dict(self, *args, **kwargs):
        self._drop_prepared()
        return super()._load_from_state_dict(*args, **kwargs)
