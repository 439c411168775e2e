"""CPU restatement of the reference's unfused (torch) softmax and rotary path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``gpt-neox_amd/`` imports this package;
it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline.

* ``torch_ref``  -- the reference's torch expressions, restated op for op.
* ``brute``      -- an independent float64 evaluation with Python/numpy loops, used
                    to pin ``torch_ref`` on small inputs.
* ``philox``     -- Philox4x32-10 and the element -> random bits assignment of the fused
                    attention-dropout kernels, in numpy; pinned by Random123's published
                    known-answer vectors, a per-element pure-Python restatement, and (on
                    the GPU) ``torch.rand``, which consumes the same block function.

Pins (tests/test_oracle_*.py): the reference ships no golden vectors, fixtures or
asserting tests for this path, so every function here is pinned by closed forms,
invariants, brute force on tiny inputs, fp64 gradcheck and -- for the rotary
pairing convention -- the installed ``transformers`` GPT-NeoX implementation.
The dropout expressions of ``torch_ref`` (``dropout_scale``, ``dropout_with_mask``,
``softmax_dropout_backward_fp32``) are pinned by fp64 autograd of the unfused expression, by
the float64 vectors ``tests/golden/dropout_*.npz`` (written from ``brute``) and, on the GPU,
by the kept entries of ``torch.nn.functional.dropout`` itself.
No function of this package is "parity unpinned".
"""
