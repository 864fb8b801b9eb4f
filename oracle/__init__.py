"""CPU oracle for the batched-decode hot path (TEST INFRASTRUCTURE ONLY).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package, and only as the checker. The product (vexel_amd) never imports it.

numerics.py wraps the C restatement in vexel_oracle.c; host_logic.py restates the
integer bookkeeping (block pool, packing, candidate trees); model.py chains them into
the reference's layer / decode drivers; quantize.py makes synthetic quantized weights.
"""
from . import numerics, host_logic, quantize, model  # noqa: F401
