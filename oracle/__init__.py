"""CPU oracle for conv2d_gw8 -- TEST INFRASTRUCTURE ONLY.

Nothing under oracle/ is part of the product.  Only tests/, the smoke check in
__graft_entry__.py and the cpu_baseline leg of bench.py may import it, and only
as the checker.  The product (spio_amd) never imports it and has no CPU path.
"""
