"""MI355X-native LRQK decode path."""
