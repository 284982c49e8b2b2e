"""Transformer factory API (ngraph/transformers/__init__.py:17-52).

Importing this package registers the HIP backends; a backend whose library
cannot be loaded is left out of `transformer_choices()`, as the reference does
for its optional GPU backends (ngraph/transformers/__init__.py:34-47).
"""
from ngraph_hip.transformers.base import (  # noqa: F401
    make_transformer, set_transformer_factory, get_transformer_factory, transformer_choices, allocate_transformer,
    make_transformer_factory, Transformer, Computation, UnsupportedTransformerException)

import ngraph_hip.transformers.hiptransform  # noqa: F401
import ngraph_hip.transformers.flexhiptransform  # noqa: F401
