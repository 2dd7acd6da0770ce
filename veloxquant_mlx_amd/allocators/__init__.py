"""VecInfer building blocks."""
