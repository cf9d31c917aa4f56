"""MI355X-native layer-wise DP core for the Galvatron search engine (host side)."""
