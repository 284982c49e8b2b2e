"""flex16: int16 mantissas with one shared exponent per tensor.

`base` mirrors ngraph/flex/base.py.  `hipflex` provides what the reference imports
from the private `autoflex.gpu` package (ngraph/flex/__init__.py:1-4): the
manager, the per-tensor entry and the 16-bit flex dtype.
"""
from ngraph_hip.flex.base import Flex, flex16, FlexEntry, FlexManager, flex_gpu_transformer_name  # noqa: F401
from ngraph_hip.flex.hipflex import HipFlexManager, HipFlexEntry, HipFlex, hipflex16  # noqa: F401
