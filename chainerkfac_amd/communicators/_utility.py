"""Buffer sizing for the packed communicator layout."""


def get_nelems(arrays):
    """Number of buffer elements for ``arrays`` (list per rank of lists of
    ``(array, triangular)``): n(n+1)/2 for a triangular n x n array, ``size``
    otherwise.  Same contract as the reference's
    chainerkfac/communicators/_utility.py:72-83."""
    nelems = 0
    for local_arrays in arrays:
        for array, triangular in local_arrays:
            if triangular:
                if array.ndim != 2 or array.shape[0] != array.shape[1]:
                    raise RuntimeError('get_nelems: not a square matrix')
                nelems += array.shape[0] * (array.shape[0] + 1) // 2
            else:
                nelems += array.numel()
    return nelems
