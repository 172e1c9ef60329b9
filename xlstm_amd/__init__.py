"""MI355X-native sLSTM forward / decode engine behind the reference's sLSTMCell API."""
__version__ = "0.1.0"
