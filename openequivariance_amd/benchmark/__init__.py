"""Benchmark and correctness harness with the reference's entry points and JSON result layout
(reference: openequivariance/benchmark/): TestBenchmarkSuite / ConvBenchmarkSuite run lists of
problems, write one JSON file per test plus metadata.json, and the helper modules keep the
reference's names.  Correctness needs a reference implementation supplied by the caller (or an
installed e3nn); nothing here computes tensor products on the CPU."""
