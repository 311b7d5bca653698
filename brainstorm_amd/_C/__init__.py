"""Stand-ins for the reference's compiled extension modules (``brt._C``)."""
