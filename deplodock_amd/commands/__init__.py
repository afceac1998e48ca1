"""Command-line front end: ``python -m deplodock_amd {compile,run} --code "<expr>"``.

Only the two commands that drive the kernel path are provided, with the
reference CLI's argument names (emmy/emmy.py:25-56, emmy/commands/compile.py,
emmy/commands/run.py).
"""
