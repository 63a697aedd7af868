"""Example models written as user-defined functions (``udf``), two-layer
networks over their compiled plans (``models``) and the benchmark driver
(``run``: ``python -m graphiler_amd.examples.run``)."""
