"""Package version (API level of the reference this build mirrors: 2.0.1)."""
__version__ = "2.0.1+mi355x.0"
