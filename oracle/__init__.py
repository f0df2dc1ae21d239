"""CPU oracle for the gradient-compression hot path.

TEST INFRASTRUCTURE ONLY.  Importable from tests/, from the smoke test and from
the benchmark's cpu_baseline leg; the product package never imports it.

  oracle.cpu       ctypes binding of liboracle.so (plain-C restatement of the
                   reference's TBQ / TernGrad / GradDrop bodies)
  oracle.ref       ctypes binding of _ref/libhpref.so (the reference's own
                   header bodies compiled for the host; optional, present only
                   where it was built from a reference checkout)
  oracle.powersgd  numpy fp64 statement of the PowerSGD phases
"""
