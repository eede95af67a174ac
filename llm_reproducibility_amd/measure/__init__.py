"""Measurement helpers of the benchmark: machine probes (libtbik_measure.so, built from probe.hip) and the summariser of
rocprofv3 output.  Nothing here is on the product path."""
