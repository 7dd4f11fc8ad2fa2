"""HIP backend of the analog linear operator: C-ABI binding, torch custom ops, autograd glue."""
