"""CPU checkers for the HIP convolution kernels.  Test infrastructure only."""
