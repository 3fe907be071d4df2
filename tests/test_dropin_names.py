"""The reference's import names resolve to this build (package onebit_sparse_mul, module onebit_sparse_cuda)."""


def test_reference_import_names():
    import onebit_sparse_mul
    from onebit_sparse_mul._semi_structured_conversions import (  # noqa: F401
        mask_creator,
        sparse_semi_structured_from_dense_cutlass,
        sparse_semi_structured_to_dense_cutlass,
    )
    from onebit_sparse_mul import BinaryLinear_2_4, binary_quant, pack_binary, dequant_desparse_tile  # noqa: F401
    import onebit_sparse_cuda
    assert hasattr(onebit_sparse_cuda, "onebit_mul")
    assert onebit_sparse_mul.cuda_binary_mul.__module__ == "onebitsparsemul_amd"
