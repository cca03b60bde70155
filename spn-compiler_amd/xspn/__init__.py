"""Pure-Python stand-in for the reference's ``xspn`` package (xspn/xspn/): the query/model
wrappers and a Cap'n Proto writer/reader for ``spflow.capnp`` that need neither pycapnp nor SPFlow."""
