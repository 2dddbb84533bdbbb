"""Test-side names for the host harness of the package (model builders, seeded inputs, device buffers)."""
from fitre_amd.harness import *  # noqa: F401,F403
from fitre_amd.harness import (Device, GpuModel, at, batch_inputs, build_alexnet, build_custom, build_lenet,  # noqa: F401
                               build_vgg11, conv_shape, he_weights, input_dims, num_classes, rel_err)
