"""CPU oracle for the gradient-compression hot path.

TEST INFRASTRUCTURE ONLY.  Importable from tests/, from the smoke test and from
the benchmark's cpu_baseline leg; the product package never imports it.

  oracle.cpu       ctypes binding of liboracle.so (plain-C restatement of the
                   reference's TBQ / TernGrad / GradDrop bodies)
  oracle.powersgd  numpy fp64 statement of the PowerSGD phases
"""
