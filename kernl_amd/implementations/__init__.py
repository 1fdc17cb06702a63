"""The three fused operators (reference: src/kernl/implementations/)."""
