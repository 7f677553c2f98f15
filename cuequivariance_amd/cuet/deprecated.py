"""Names the reference removed from its API and keeps only as stubs that refuse to be built
(``cuequivariance_torch/primitives/deprecated.py:26-168``): importing them works, constructing one raises ``ImportError`` with
the replacement to use."""

__all__ = ["TensorProduct", "EquivariantTensorProduct", "SymmetricTensorProduct", "IWeightedSymmetricTensorProduct"]


class _Removed:
    _instead = ""

    def __init__(self, *args, **kwargs):
        raise ImportError(f"{type(self).__name__} has been removed.\n{self._instead}")


class TensorProduct(_Removed):
    _instead = ("Use SegmentedPolynomial: poly = cue.SegmentedPolynomial.eval_last_operand(descriptor); "
                "cuet.SegmentedPolynomial(poly, method='uniform_1d' | 'fused_tp' | 'indexed_linear', math_dtype=...), or the modules "
                "ChannelWiseTensorProduct / FullyConnectedTensorProduct.")


class EquivariantTensorProduct(_Removed):
    _instead = ("Use SegmentedPolynomial on the polynomial of the descriptor: cuet.SegmentedPolynomial(e.polynomial, method=..., "
                "math_dtype=...); layouts are changed with TransposeIrrepsLayout, or use the modules ChannelWiseTensorProduct, "
                "FullyConnectedTensorProduct, Linear, SymmetricContraction.")


class SymmetricTensorProduct(_Removed):
    _instead = ("Use SegmentedPolynomial with the input repeated in the operations of the polynomial (one polynomial holds all "
                "degrees), or the module SymmetricContraction.")


class IWeightedSymmetricTensorProduct(_Removed):
    _instead = ("Use SegmentedPolynomial with the weights as an indexed input: f([weights, x], input_indices={0: indices}), or the "
                "module SymmetricContraction.")
