"""Graph-rewrite passes and hipGraph capture (reference: src/kernl/optimizer/)."""
