"""Recurrent layers composed from ``AnalogLinear``."""
