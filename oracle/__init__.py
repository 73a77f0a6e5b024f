"""CPU oracle for the k-quant path.  Test infrastructure only: the product never imports this."""
