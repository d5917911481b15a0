"""TEST INFRASTRUCTURE: CPU oracle for the int8 pseudo-gradient compression path.

Only tests/, ``__graft_entry__.smoke()`` and bench.py's ``cpu_baseline`` leg may import
this package.  The product package (``prime_amd``) never does.
"""
