"""MI355X-native two-layer MACE inference engine behind the symmetrix API."""
