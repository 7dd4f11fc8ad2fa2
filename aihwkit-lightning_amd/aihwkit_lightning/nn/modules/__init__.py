"""Analog modules."""
