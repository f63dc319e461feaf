"""MI355X-native operator backend behind BackendBench's directory-backend boundary."""

__version__ = "0.1.0"
