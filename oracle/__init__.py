"""CPU oracle for the permutohedral encoding: TEST INFRASTRUCTURE, not product code.

Only the tests, ``__graft_entry__.smoke()`` and the CPU-baseline leg of ``bench.py`` import this
package, and only as the checker / the reported CPU baseline.  The shipped package
(``permutohedral_encoding_amd``) never imports it and has no CPU fallback.

``oracle.api`` is a ctypes binding over ``libpenc_oracle.so`` (built from ``penc_oracle.cpp`` by
``make -C oracle``).
"""
