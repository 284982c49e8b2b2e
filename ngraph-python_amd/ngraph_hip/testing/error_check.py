"""assert_allclose with per-transformer default tolerances
(ngraph/testing/error_check.py:26-83)."""
import numpy as np

import ngraph_hip.transformers as ngt


def assert_allclose(actual, desired, rtol=1e-07, atol=0, transformer_overwrite=True, **kwargs):
    """np.testing.assert_allclose widened to the current transformer's default tolerance."""
    if transformer_overwrite:
        factory = ngt.get_transformer_factory()
        cls = ngt.Transformer.transformers.get(getattr(factory, "name", None))
        if cls is not None:
            t_atol, t_rtol = cls.get_default_tolerance(np.asarray(desired))
            atol = max(atol, t_atol)
            rtol = max(rtol, t_rtol)
    return np.testing.assert_allclose(actual, desired, rtol=rtol, atol=atol, **kwargs)
