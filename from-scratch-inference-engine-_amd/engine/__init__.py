"""The step function, the scheduler above it, and the entry points."""
