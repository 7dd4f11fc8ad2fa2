"""Configuration objects read by the analog layers."""
