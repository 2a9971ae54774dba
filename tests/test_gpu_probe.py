"""The matrix-core probe of the benchmark (csrc/sc_probe.hip): its fp4 GEMM tile with threshold and count gives
exactly the counts of the bit-serial definition - OR over the members of a group of the AND of activation and weight
bits (sc.cpp:12-259) - for one and for several slices, so what the probe times is the forward's arithmetic."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_mfma_slice_counts_equal_the_or_of_ands():
    from geo_amd import capi
    a, b, a_bits, b_bits = capi.probe_mfma_operands(3, 2, seed=1, p_a=1 / 64, p_b=1 / 32)
    # one slice per workgroup: workgroup w multiplies A tile w with B tile 0
    got = capi.probe_mfma_slices(2, a, b, workgroups=3, slices=1).cpu()
    sums = torch.einsum("wmk,jk->wmj", a_bits.float(), b_bits[0].float())
    want = (sums > 0).int()
    assert torch.equal(got, want)
    assert 0.05 < want.float().mean().item() < 0.95      # both outcomes occur
    # five slices of the same operands (modes 0 - 2 keep their tiles): five times the count
    got5 = capi.probe_mfma_slices(2, a, b, workgroups=3, slices=5).cpu()
    assert torch.equal(got5, 5 * want)
