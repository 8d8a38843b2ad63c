"""CPU oracle for the column-vector-sparse SpMM/SDDMM path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this
package; only the tests, the smoke check and the CPU-baseline leg of the
benchmark do, and only as the checker.

`numpy_oracle` restates the reference's host loops with numpy (bit-identical
to the C restatement because the order of fp32 additions per output element is
the same); `c_oracle` loads `libvsoracle.so`, built from `vs_oracle.c`.
"""
