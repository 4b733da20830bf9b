"""Files meant to be copied into a fairscale checkout (they do not import this package)."""
