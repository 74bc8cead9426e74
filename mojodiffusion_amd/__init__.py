"""MI355X-native SageAttention-style quantized SDPA behind the serenitymojo
attention call surface."""
