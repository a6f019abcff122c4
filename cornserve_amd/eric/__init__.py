"""Host-side mirror of the slice of Cornserve's Eric executor that surrounds the encoder forward pass."""
