"""offload_adam_amd: Adam with host-offloaded state, MI355X-native kernels."""

__version__ = "0.1.0"
