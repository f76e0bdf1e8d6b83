"""Constants and the operator-registration helper, source compatible with upstream
``stickbreaking_attention/utils.py`` (``custom_op`` :20-39, ``_dispatch`` :12-17)."""
import math
from typing import Callable, Iterable, Optional, Sequence, Union

import torch

PACKAGE_NAME = "stickbreaking_attention"
log2 = math.log(2)
inv_log2 = 1 / log2


def custom_op(name: str, mutates_args: Union[str, Iterable[str]],
              device_types: Optional[Union[str, Sequence[str]]] = None, schema: Optional[str] = None) -> Callable:
    """Register ``func`` as the PyTorch operator ``stickbreaking_attention::<name>`` and return a
    callable that goes through the registered operator only while ``torch.compile`` is tracing
    (where an opaque operator is needed) and calls ``func`` directly otherwise (no dispatcher
    overhead in eager mode) -- the arrangement upstream uses for its Triton launchers."""
    qualified = f"{PACKAGE_NAME}::{name}"

    def wrap(func: Callable) -> Callable:
        registered = torch.library.custom_op(qualified, func, mutates_args=mutates_args,
                                             device_types=device_types, schema=schema)

        def run(*args, **kwargs):
            if torch.compiler.is_compiling():
                return registered(*args, **kwargs)
            return func(*args, **kwargs)

        run.registered = registered
        run.__name__ = getattr(func, "__name__", name)
        return run

    return wrap
