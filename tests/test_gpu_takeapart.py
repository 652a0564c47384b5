"""The take-apart timing of a fused pair (python -m hfuse_amd.takeapart) on the product library."""
import pytest


@pytest.mark.gpu
def test_takeapart_row_of_the_histogram_pair(cuda):
    from hfuse_amd import takeapart
    row = takeapart.run("histc_maxpool", rounds=1, rotations=1)
    us = row["us"]
    assert set(us) == {"native_a", "native_b", "back_to_back", "shipped", "partition", "shipped_a_alone", "shipped_b_alone",
                       "partition_a_alone", "partition_b_alone"}
    assert row["library"] == "libhfuse_gfx950.so" and row["pair"] == "histc_maxpool"
    assert all(v > 0 for v in us.values())
    # a kernel alone inside the fused kernel is no slower than the pair, and the launch of both natives no faster than either
    assert us["shipped_a_alone"] < us["shipped"] * 1.05 and us["shipped_b_alone"] < us["shipped"] * 1.05
    assert us["back_to_back"] > max(us["native_a"], us["native_b"]) * 0.95
