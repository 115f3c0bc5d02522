"""MI355X-native stage executor behind the JaxPP pipeline-parallel API."""
__version__ = "0.1.0"
