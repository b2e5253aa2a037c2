"""CPU oracle for the Connect6 policy/value forward path.

TEST INFRASTRUCTURE ONLY.  Nothing in ``connect6_amd`` imports this package.
Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may use it, and only as the checker.

Contents
--------
``torch_ref``   plain-PyTorch fp32 restatement of the reference forward pass,
                the grouped history forward, ``mask_logits``, inverse-CDF
                sampling, and the D4 board/action maps.
``conv_ref.c``  brute-force double-precision direct convolution of the same
                network in plain C (no library routine), used to pin
                ``torch_ref`` on small inputs.
``cref``        ctypes binding of ``conv_ref.c``.
``env_ref``     restatement of the batched environment step (``VectorConnect6.step``
                with its local win check) plus an independent scalar game that pins it.

Pinning status of every oracle function is listed in the headers of ``torch_ref`` and ``env_ref``.
"""
