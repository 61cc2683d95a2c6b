"""Host simulation of the GPU kernels: test infrastructure, nothing in the package uses it.

The package's own ``.hip`` sources are compiled for the CPU (``build.py``) against a stand-in
``hip/hip_runtime.h`` and a small runtime (``hostsim.cpp``: every GPU lane a fiber; ``order.cpp``: vector
clocks for streams and events).  What the pieces are for:

``sim.py``            the simulated library bound like the real one; ``sim.guard(t)``: a tensor that ends at an
                      inaccessible page (``HOSTSIM_GUARD_SIDE=front``: that starts right after one)
``mode.py``           ``FLEXTRAIN_HOSTSIM=1 python -m pytest tests -m gpu``: the GPU parity tests on the simulation;
                      device tensors are guarded, uninitialised memory reads as NaN / -1, streams and events
                      carry clocks and an unordered overlapping access on two streams fails the enqueuing call
``HOSTSIM_LANE_ORDER``  ``descending``: the lanes of a workgroup run in descending order between barriers
                      (a missing barrier shows in one of the two orders)
``hostsim_set_dma_eager(1)``  loads into LDS land at their issue instead of as late as the lane's counted
                      waits allow (the default); the GEMM tests run at both extremes
``bench_shapes.py``   ``python -m tests.hostsim.bench_shapes``: the bandwidth-bound kernels at bench.py's exact shapes
``bench_dry_run.py``  ``python -m tests.hostsim.bench_dry_run``: bench.py itself over launches that return at once
``skip_in_simulation.txt`` / ``slow_in_simulation.txt``  GPU tests without meaning there / left to the run by hand
"""
