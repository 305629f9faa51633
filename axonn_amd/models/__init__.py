"""Model-level glue over the Linear kernels (axonn/models in the reference)."""
