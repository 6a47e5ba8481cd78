"""Import-path alias: `from benchmark.utils.utils import ...` as in the reference's benchmark scripts."""
