"""MI355X-native one-GPU inference runtime for Qwen3 dense models."""
