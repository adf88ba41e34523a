"""CPU oracle for the attention path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product (the HIP library, the extension, the ``flash_attn_v100``
package) may import or call anything in this directory.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and
only as the checker.
"""
