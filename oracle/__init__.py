"""TEST INFRASTRUCTURE ONLY — CPU restatement of the reference's mops torch-backend semantics.

Nothing in the product package imports this directory.  It may be imported by tests/, by
__graft_entry__.smoke() and by bench.py's cpu_baseline leg, always as the checker / baseline and never
as the implementation being measured or shipped.
"""
