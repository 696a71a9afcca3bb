"""MI355X-native implementation of the MCCNN point-cloud custom-op path.

Sub-modules
    tfg_custom_ops  the eight op entry points of the reference's native package,
                    on torch tensors, dispatching into libmccnn_hip.so
    custom_ops      object-level adapters of those ops (point clouds, grids and
                    neighbourhoods instead of raw tensors)
    pc              thin counterparts of the reference's callers (grid,
                    neighbourhood, sampling, hierarchy)
    layers          Monte-Carlo / kernel-point convolutions and pooling built on
                    the ops
    blocks, models  1x1 convolution, residual blocks, the classification network
    io, kernel_points, train_classification
                    file loaders, kernel-point layouts, the training loop
    synthetic       seeded input generators for the benchmark configurations

Importing this package does not load the HIP library; the first op call does,
and it raises if the library has not been built.
"""
__all__ = ["synthetic"]
