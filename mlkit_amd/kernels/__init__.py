"""Launch wrappers over the C ABI, one module per reference kernel module."""
