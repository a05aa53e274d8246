"""TEST INFRASTRUCTURE, NOT PRODUCT CODE: CPU restatements of the reference's
paged KV-cache data movement. Only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg import this package; lmserve_amd/ never does."""
