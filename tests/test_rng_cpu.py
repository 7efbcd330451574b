"""Known-answer test of the Philox4x32-10 restatement the GPU masks are checked against
(vectors from the Random123 distribution's kat_vectors: philox4x32 10)."""
from nmtgminor_amd._rng import philox4x32_10, philox_keep_mask_reference


def test_philox_known_answers():
    assert philox4x32_10([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert philox4x32_10([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert philox4x32_10([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]) == \
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]


def test_keep_mask_is_a_function_of_the_element_index():
    a = philox_keep_mask_reference(42, 8, 0, 64, 0.5)
    b = philox_keep_mask_reference(42, 8, 16, 16, 0.5)
    assert a[16:32] == b and 10 < sum(a) < 54
    assert philox_keep_mask_reference(42, 12, 0, 64, 0.5) != a
