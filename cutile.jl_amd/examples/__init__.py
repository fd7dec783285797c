"""Host harnesses that mirror the reference's examples/*.jl one to one: each module has the
example's ``prepare`` / ``run`` / ``metric`` functions (same keyword names and defaults) and
launches the kernels through the C ABI where the reference uses ``@cuda backend=cuTile``.

``verify`` is not here: checking needs a CPU restatement of the example's reference math,
which lives with the tests (``oracle/``), never in the product.
"""
