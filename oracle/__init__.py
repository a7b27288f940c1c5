"""CPU oracle of the deformable-convolution hot path.  Test infrastructure only: nothing in the
shipped package imports this."""
