"""CPU oracle for the compiled-op path: test infrastructure only.

Importable from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg; the product
package never imports it.
"""
