"""Custom-op adapters over the C-ABI kernels (stateless)."""
