"""MI355X-native fused optimizer steps behind the grokking_optimizers API."""
