"""CPU oracle of the multi-step spiking-neuron path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``spikingjelly_amd/`` imports this package; only ``tests/``, ``bench.py``'s
``cpu_baseline`` leg and ``__graft_entry__.smoke()`` do, as the checker.  It restates the
reference's torch backend (SpikingJelly, ``spikingjelly/activation_based``) on the CPU:

``neuron_oracle``   torch-ops restatement, op for op, of ``functional/neuron.py`` (``voltage_reset``
                    :225-228, ``if_step`` :310-312, ``lif_charge`` :849-852, ``lif_step`` :931-933,
                    ``plif_step`` :1290-1297), ``surrogate.py`` (``heaviside`` :60, ``sigmoid`` :769-851,
                    ``atan`` :1247-1330, ...), the step loop + ``torch.stack`` of ``base.py:594-607`` /
                    ``neuron/base_node.py:443-464`` and the mixed-precision recipe of the reference's
                    own test (``test/activation_based/test_triton_neuron.py:212-247``).  Gradients come
                    from torch autograd through those ops, as in the reference.
``bptt_oracle``     the closed-form BPTT recurrence in numpy float64 (derived from
                    ``cuda_kernel/neuron_kernel/multi_step/base.py:293-409``, ``lif.py:89-102``,
                    ``plif.py:143-203``).
``bitpack_oracle``  numpy restatement of ``triton_kernel/compress.py:19-44``.
``c_oracle``        ctypes binding of ``sj_oracle.c``, a plain-C scalar restatement of the same
                    forward, BPTT and bit-packing (built by ``oracle/Makefile``).

How each function is pinned (tests/test_oracle_*.py): the hand-checkable 4x4 dyadic input of
the reference's ``test_triton_neuron.py:1207-1216`` with expected values from exact rational
arithmetic (``tests/golden/dyadic_4x4.json``); closed forms (T=1, zero-input decay, the IF
soft-reset rate-coding identity, hard-reset invariants); the surrogate finite-difference contract
of ``test_neuron_kernel_surrogate_contract.py:25-44`` and the values at 0; BPTT recurrence ==
autograd of the restated ops in float64 == central finite differences of the smooth (primitive
surrogate) network; bit-packing == ``numpy.packbits(bitorder='little')`` plus the reference's 2x3
and 17-element round trips; torch oracle == C oracle bit for bit on random fp32 inputs.
"""
