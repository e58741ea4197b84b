"""TEST INFRASTRUCTURE: CPU oracle for the ROIAlign path.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package.  The product (mobulaop_amd) never does.
"""
