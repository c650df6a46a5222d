"""CPU oracle for the SPION sparse-attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``spion_amd/`` may import this
package; it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline.
"""
