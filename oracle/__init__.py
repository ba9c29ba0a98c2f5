"""CPU oracle for the quantized Dense / EinsumDense path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``keras_amd/`` may import this
package; it exists so that ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` have something independent to check the
HIP path against.
"""
