"""CPU oracle for the voxel scatter-reduction path.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py``.  Nothing under ``torchex_amd/``
imports it.

``c_oracle``     ctypes binding of ``scatter_oracle.c`` (lane-exact restatement
                 of the reference kernels + spec functions over unsorted ids).
``torch_oracle`` the same operators written with ``torch.scatter_reduce`` /
                 ``index_add`` on CPU tensors; used as an independent library
                 cross-check of the C oracle and as the timed CPU baseline.
"""
