"""CPU oracle for the Qwen2.5-VL vision-tower hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this
directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may, and there only as the checker.

Modules
-------
``vit_oracle``  plain-PyTorch (CPU, eager) restatement of the vision tower
                forward; gradients come from ``torch.autograd``.
``sp_oracle``   numpy / pure-Python restatement of the ragged
                sequence-parallel index arithmetic (cuts, split, pad, gather).

Pinning status (what each function is checked against, other than itself):
see the module docstrings; every function there names its check or says
"parity unpinned".
"""
