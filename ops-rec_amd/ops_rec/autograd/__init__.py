"""Attaches the autograd formula of the HSTU attention operators when the package is imported.

This package carries exactly one plug-in, ``hstu_v1_autograd``; it is imported by name and its
``register_autograd()`` is called once.  The reference walks its ``autograd`` directory and registers
whatever module it finds there (ops_rec/autograd/__init__.py:26-48); the observable contract kept here is
the same: importing ``ops_rec`` must not fail because a formula could not be attached (the forward
operators stay usable, a message goes to the log), and ``__all__`` names the plug-ins that are active.
"""

import logging

_log = logging.getLogger(__name__)

__all__: list = []


def _attach(name: str) -> None:
    """Import plug-in ``name`` of this package and run its ``register_autograd()``; log instead of raising."""
    try:
        module = __import__(f"{__name__}.{name}", fromlist=[name])
        module.register_autograd()
    except Exception as err:  # noqa: BLE001  (an import of ops_rec must survive a broken plug-in)
        _log.warning("autograd formula '%s' is not active (%s: %s)", name, type(err).__name__, err)
        return
    __all__.append(name)


_attach("hstu_v1_autograd")
