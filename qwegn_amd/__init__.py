"""qwegn_amd: MI355X-native quantized matmul path (libqwhip) and its host bindings."""
