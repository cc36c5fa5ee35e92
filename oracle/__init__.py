"""TEST INFRASTRUCTURE ONLY: the CPU oracle for the QLoRA quantized-linear path.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg
may import this package.  The product package (``xorl_amd``) never does: its
ops raise when the HIP library is missing.

Three layers:

* ``oracle.cdecode`` -- ctypes binding of ``xq_oracle.c`` (plain C restatement
  of the reference codecs, built by ``oracle/Makefile``).
* ``oracle.decode_np`` -- an independently written numpy twin of the decoders,
  used to cross-check the C file (table-driven instead of bit-built).
* ``oracle.recipe`` -- the reference's forward/backward *recipe* in torch CPU
  ops (what ``QLoRALinear.forward`` and the grouped LoRA MLP compute, with
  their rounding points), plus fp32-accumulated variants the tolerance tests
  compare against.
"""
