"""CPU checkers for the HIP backend (test infrastructure only).

``oracle.api``  -- ctypes front end of ``repdl_oracle.c`` with the reference's
                   operator signatures (torch CPU tensors in and out).
``oracle.ref``  -- loader of RepDL's own C++ CPU backend when it has been
                   compiled into ``oracle/_ref`` (see ``oracle/build.py``).
Only tests, the smoke check and the benchmark's cpu_baseline leg import this.
"""
