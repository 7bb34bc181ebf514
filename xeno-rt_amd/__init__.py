"""MI355X-native model library for the Llama / Qwen3 dense decoder."""
