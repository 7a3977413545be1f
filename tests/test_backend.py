"""The KokkosBackend-shaped front door: signature parsing and catalogue checks (CPU only)."""
import pytest

from lapis_amd.KokkosBackend import KokkosBackend, _public_functions

SPMV_NOALLOC = """
#sparse = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
module {
  func.func @spmv(%A: tensor<?x?xf64, #sparse>, %x: tensor<?xf64>, %y: tensor<?xf64>) -> tensor<?xf64> {
    %0 = linalg.matvec ins(%A, %x: tensor<?x?xf64, #sparse>, tensor<?xf64>) outs(%y : tensor<?xf64>) -> tensor<?xf64>
    return %0 : tensor<?xf64>
  }
}"""

PCG = """
module {
  func.func private @spmv(%A: tensor<?x?xf64, #sparse>, %x: tensor<?xf64>, %ydst: tensor<?xf64>) -> tensor<?xf64> { }
  func.func private @dot(%x: tensor<?xf64>, %y: tensor<?xf64>) -> f64 { }
  func.func @pcg(%A: tensor<?x?xf64, #sparse>, %b: tensor<?xf64>, %dinv: tensor<?xf64>, %tol: f64, %maxiter: index) -> (tensor<?xf64>, index, f64) { }
}"""


def test_public_functions_skip_private_helpers():
    assert [f[0] for f in _public_functions(PCG)] == ["pcg"]
    assert [f[0] for f in _public_functions(SPMV_NOALLOC)] == ["spmv"]


def test_bind_accepts_the_path_and_renames_main():
    b = KokkosBackend(decompose_tensors=True)
    assert b.bind(SPMV_NOALLOC) == ["spmv"]
    assert b.bind(PCG) == ["pcg"]
    torch_mv = "func.func @main(%arg0: tensor<5x5xf64, #sparse>, %arg1: tensor<5xf64>) -> tensor<5xf64> { }"
    assert b.bind(torch_mv) == ["lapis_main"]


BSPMM = """
#csrv = #sparse_tensor.encoding<{ map = (d0, d1, d2) -> (d0 : dense, d1 : compressed, d2 : dense), posWidth = 32, crdWidth = 32}>
module {
  func.func @pte_local_bspmm(%A: tensor<?x?x?xf32, #csrv>,
    %B: tensor<?x?x?xf32>) ->  tensor<?x?x?xf32>
  { }
  func.func @print_csrv(%A: tensor<?x?x?xf32, #csrv>)
  { }
}"""


def test_bind_takes_the_batched_csrv_product_and_sets_its_print_helper_aside():
    # shape of the module in examples/bspmm.py:10-60
    b = KokkosBackend(decompose_tensors=True)
    assert b.bind(BSPMM) == ["pte_local_bspmm"]
    assert b.unbound == ["print_csrv"]


def test_bind_rejects_what_the_module_does_not_implement():
    b = KokkosBackend(decompose_tensors=True)
    with pytest.raises(Exception, match="Lowering to Kokkos dialect failed"):
        b.bind("func.func @gemm(%a: tensor<?x?xf64>, %b: tensor<?x?xf64>) -> tensor<?x?xf64> { }")
    with pytest.raises(Exception, match="Lowering to Kokkos dialect failed"):
        b.bind("func.func @spmv(%x: tensor<?xf64>) -> tensor<?xf64> { }")  # right name, wrong signature
    with pytest.raises(Exception, match="decompose_tensors"):
        KokkosBackend().bind(SPMV_NOALLOC)
    with pytest.raises(Exception):
        b.bind("module { }")


def test_constructor_mirrors_the_reference():
    b = KokkosBackend(decompose_tensors=True, parallel_strategy="dense-outer-loop", index_instance=2, num_instances=3)
    assert b.package_name == "lapis_package_2" and b.parallel_strategy == "dense-outer-loop"
    assert KokkosBackend().package_name == "lapis_package"
