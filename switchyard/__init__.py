"""The reference's module path for the kernels of the MoE layer, served by switchyard_amd.

Only `switchyard.kernels` exists here: the one-GPU MoE layer is the path this build replaces.
Code written against the reference (`from switchyard import kernels`) runs on the gfx950
library unchanged."""
