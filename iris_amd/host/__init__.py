"""Host-side pieces of the Iris context: HIP runtime access, logging, the symmetric heap."""
