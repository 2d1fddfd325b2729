"""Autograd plug-ins: every module here that exposes ``register_autograd()`` is imported and
registered when the package is imported; a failure in one module is logged and does not stop
the others (ops_rec/autograd/__init__.py:26-48 in the reference)."""

import importlib
import logging
import pkgutil

logger = logging.getLogger(__name__)

__all__: list = []


def _register_modules() -> None:
    for _, mod_name, is_pkg in pkgutil.iter_modules(__path__):
        if is_pkg:
            continue
        try:
            mod = importlib.import_module(f"{__name__}.{mod_name}")
        except Exception as exc:  # noqa: BLE001
            logger.warning("ops_rec.autograd: failed to import '%s': %s", mod_name, exc)
            continue
        fn = getattr(mod, "register_autograd", None)
        if fn is None:
            logger.warning("ops_rec.autograd: module '%s' has no register_autograd(), skipping", mod_name)
            continue
        try:
            fn()
        except Exception as exc:  # noqa: BLE001
            logger.warning("ops_rec.autograd: register_autograd() in '%s' failed: %s", mod_name, exc)
            continue
        __all__.append(mod_name)


_register_modules()
