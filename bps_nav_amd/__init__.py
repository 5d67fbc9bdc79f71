"""MI355X-native batch environment-step engine with the bps_sim / bps_pytorch surface."""
