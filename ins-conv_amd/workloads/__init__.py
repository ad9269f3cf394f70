"""Seeded synthetic inputs and the network definition of the five benchmark workloads.

`scenes` generates the voxel scenes, `netdefs` builds the U-Net of the reference's usage example
(model.py:8-26).  bench.py, the smoke test and the test suite all take their inputs from here, so
that what is measured and what is checked are the same data.
"""
