"""CPU oracle for the paged-decode hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under this directory is part of the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  The product path
(``nanovllm_jax_amd``) never imports it and has no CPU fallback.
"""
