"""Python side of the HIP kernel library: loading (and building at first use) and checked calls."""
