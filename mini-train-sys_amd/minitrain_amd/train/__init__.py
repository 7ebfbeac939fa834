"""Training-step recipe around the host model."""
