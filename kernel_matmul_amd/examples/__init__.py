"""Small end-to-end uses of the operators (the counterpart of the reference's ``examples/``)."""
