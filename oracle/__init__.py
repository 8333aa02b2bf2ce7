"""CPU oracle for the hipml full-attention hot path (test infrastructure only).

`oracle.binding` wraps ``libhipml_oracle.so`` (built from ``hipml_oracle.c``)
with numpy-friendly functions.  Nothing under ``hipml_amd`` may import this
package: it is the checker, never the product.
"""
