"""ORACLE — TEST INFRASTRUCTURE ONLY (see eager.py and tde_oracle.c for what is restated from where).
The product package torch_dist_ext_amd never imports this."""
