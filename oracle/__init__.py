"""CPU oracle for the MoE hot path — TEST INFRASTRUCTURE, not part of the product.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this package.
`torch_oracle` restates the reference's torch path with plain torch CPU operators; `c_oracle` binds
the scalar C restatement in moe_oracle.c.
"""
