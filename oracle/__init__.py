"""Checker for the HIP feature transformer.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this directory; it is used by tests/,
by __graft_entry__.smoke() and by bench.py's cpu_baseline leg.

  oracle.cpu        ctypes front end of libnnueft_oracle.so (nnueft_oracle.c), numpy in / numpy out
  oracle.ref_torch  the reference's CPU path restated with the same torch library calls
  oracle.loader_ref ctypes front end of _ref/libtraining_data_loader_ref.so (the reference's own
                    C++ encoder, compiled from the reference sources by the Makefile here)
"""
