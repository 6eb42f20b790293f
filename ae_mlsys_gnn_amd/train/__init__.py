"""Training drivers on the fused operators: the command lines and result rows of the reference's
script/train/*.py, with the whole graph pipeline (self-loops, COO -> CSR, CSR -> CSC, schedules)
on the device and data read from local files or generated at the published shapes."""
