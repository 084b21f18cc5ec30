"""Python convenience layer over sparseops_backend (mirrors the reference's python/ package)."""
