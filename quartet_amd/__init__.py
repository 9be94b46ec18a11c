"""MI355X-native implementation of Quartet's MXFP4 quantized-linear hot path."""
