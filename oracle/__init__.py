"""CPU restatement of the reference's fp8 action-inference path (TEST INFRASTRUCTURE ONLY).

This package is the checker, never the product: only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` may import it.  Nothing under ``tybok_amd/`` does.

Everything here is plain ``torch`` on the CPU, written from the reference's eager torch path
(file:line cited per function).  Modules:

* :mod:`oracle.fp8`      -- e4m3fn code table, software RNE encoder, per-row weight quantisation
* :mod:`oracle.ops`      -- fp8-weight linear, gated FFN, norms, RoPE, masks, attention, time embedding
* :mod:`oracle.smolvla`  -- SmolVLA-shaped model (prefix embed, prefill, expert denoise loop)
* :mod:`oracle.pi05`     -- pi0.5-shaped model
* :mod:`oracle.inputs`   -- the seeded synthetic inputs of the five benchmark configurations

Parity pinning status (what fixes each function besides its own formula):

* ``fp8``: all 256 codes brute-forced against the e4m3fn definition and torch's own cast; the
  encoder is cross-checked against torch's ``.to(float8_e4m3fn)``; quantisation invariants of
  ``docs/fastWAM_weight_quantization.md:26-30`` (re-quantisation byte-exact, error <= 16/448).
* ``ops``: closed forms / fp64 brute force on tiny inputs / invariants (``tests/test_oracle_*``).
* ``smolvla`` / ``pi05`` end-to-end wiring: golden vectors written once from the reference's own
  torch modules by ``tests/golden/make_golden.py`` (``tests/golden/*.npz``).
"""
