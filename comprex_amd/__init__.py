"""MI355X-native implementation of ComprEx's gradient-compression hot path."""
