"""Host-side logic that needs no GPU: context-length checks of the decode loop."""
import pytest

from rptc_kernels.llama_decode import LlamaShape, check_context


def test_greedy_decode_rejects_a_context_that_overruns_the_caches():
    shape = LlamaShape(layers=1, d_model=256, heads=4, d_ff=704, vocab=1000, max_len=640)
    check_context(shape, 512, 128)              # positions 0..638
    check_context(shape, 512, 129)              # positions 0..639: the last one the caches hold
    with pytest.raises(ValueError, match="max_len"):
        check_context(shape, 512, 130)
    with pytest.raises(ValueError):
        check_context(shape, 0, 4)
    with pytest.raises(ValueError):
        check_context(shape, 4, 0)
