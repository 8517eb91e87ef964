"""Test infrastructure: CPU restatements of the reference's quantized-linear
path.  Never imported by the shipped package (bitween_amd)."""
