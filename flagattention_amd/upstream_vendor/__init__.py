"""Files meant to be copied into an upstream FlagAttention checkout (not imported by this package)."""
