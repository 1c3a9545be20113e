"""pipec for gfx950: pack separately compiled HIP stages into ``.plink`` containers, check
their provides/needs contracts, solve LDS / wave / counter resources, generate the glue
and LTO-link everything into one code object.

Module map (what each replaces in the reference's ``pipec/src/pipec2``):
``clauses``  model.py's clause registry and error types;  ``plink``  canonjson.py +
container.py;  ``gfx950``  profile.py;  ``manifest``  schema.py;  ``channels``
protocol.py;  ``solver``  solve.py;  ``glue``  stubgen.py + dispatchgen.py;
``linker``  link.py;  ``pack``  pack/;  ``launcher``  launcher.py;  ``cli``  cli.py.
"""
from .clauses import ClauseFailure, PipeLinkError, register_clause  # noqa: F401
