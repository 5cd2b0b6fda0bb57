"""Timing harnesses for the SparseDrop HIP kernels (run as ``python -m benchmark.<name>`` from
``sparse-dropout_amd/``).  Counterparts of the reference's ``benchmark/`` scripts; they print tables
instead of drawing plots."""
