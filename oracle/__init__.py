"""TEST INFRASTRUCTURE - not part of the product.

`oracle.cpu` wraps liboracle_cpu.so (oracle/cpu_path.c: the restatement of the
reference's CPU execution of the five kernels); `oracle.ttir_lanes` is an
independent lane-by-lane interpreter of TTIR text.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package.
"""
