"""TEST INFRASTRUCTURE: CPU oracle for the MoE all-to-all dispatch/combine path.

Nothing under this package is part of the product.  It may be imported only by
``tests/``, by ``__graft_entry__.smoke()`` and by the CPU-baseline leg of
``bench.py`` -- as the checker, never as the thing measured as the GPU path.
"""
