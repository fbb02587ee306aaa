"""MI355X-native backend for the AutoRT / Antares operator surface."""
__version__ = '0.1.0'
