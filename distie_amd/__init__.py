"""MI355X-native inference engine for the Qwen2 dense decoder."""
