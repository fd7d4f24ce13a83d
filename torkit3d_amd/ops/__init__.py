"""Point-cloud operators with the API of the reference's ``torkit3d.ops`` package:
one module per op, same module names, function names, argument order, defaults and
return order (``torkit3d/ops/*.py``). Like the reference's, this package file
imports nothing, so ``torkit3d_amd.ops.ball_query`` is the module and
``torkit3d_amd.ops.ball_query.ball_query`` the function."""
