"""Small helpers kept from the reference (gear/utils.py:13-23); the HDF5 / download helpers of
the reference need network access and h5py and are not part of this build."""
import os
import pathlib
import socket
from typing import Union


def ensure_path(path: Union[str, pathlib.Path]) -> None:
    path = pathlib.Path(path)
    if not path.parent.exists():
        os.makedirs(path.parent)


def get_local_node_hashed_int32() -> int:
    from .config import KEY_T_RANGE
    return hash(socket.gethostname()) % KEY_T_RANGE
