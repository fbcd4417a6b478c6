"""The tolerances of the engine-against-plain comparisons, in one place: the GPU tests apply them and
tests/test_tolerances.py shows on the CPU that they can fail (a forward pass with a plausible mistake
exceeds them) and that bfloat16 rounding alone stays well inside them."""

# float32: rounding of a few hundred float32 operations, relative to max(1, largest |logit|)
F32_TOL = 2e-4
# bfloat16: activations are rounded to 8 bits of mantissa after every op; relative to the largest |logit|
BF16_REL_WORST, BF16_REL_MEAN = 0.06, 0.012


def bf16_within(worst: float, mean: float, scale: float) -> bool:
    return worst <= BF16_REL_WORST * scale and mean <= BF16_REL_MEAN * scale


def sharp_std(hidden_size: int) -> float:
    """The width of random matrices at which queries and keys of a model ``hidden_size`` wide come out
    about 0.8 wide, so that scores spread and attention is peaked (0.1 at 64, 0.02 at 1,536)."""
    return 0.8 / hidden_size ** 0.5
