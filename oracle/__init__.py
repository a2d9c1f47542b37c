"""CPU oracle for the octree sparse-convolution path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this directory: it exists so that the
tests, the smoke check and the benchmark's ``cpu_baseline`` leg can check (and
time) a CPU restatement of the reference algorithm next to the HIP path.

* ``octree_ref``  - Morton keys, octree build, neighbour tables (numpy, int64).
* ``conv_ref``    - conv / deconv / depth-wise conv forward, data-gradient and
                    weight-gradient (numpy fp64 literal definition, plus a
                    torch-CPU restatement of the chunked gather->mm->scatter
                    algorithm used as the timed CPU baseline).

Pinning status (what each function is checked against, see tests/test_oracle*.py):

* xyz2key / key2xyz      : closed-form bit interleave, round trip, literal keys
                           of the reference's 3-point test, every ``key`` array
                           held by the reference's fixtures.
* build_octree           : the reference's fixtures test_001..005.npz and
                           batch_45.npz (key, child, nnum, nnum_nempty, leaf
                           normals) and the literal 3-point case.
* construct_neigh        : batch_45.npz ``neigh`` (both branches), branch
                           agreement at depth 3, brute-force key search.
* get_neigh / remap      : closed forms (stride-2 '222' rows == 8p+j),
                           brute-force search on non-empty keys.
* search_key             : search_key.npz.
* conv / deconv / dwconv : torch.nn.functional.conv3d / conv_transpose3d on a
                           full layer, adjoint identities, pure-Python brute
                           force on tiny inputs.  The reference's own golden
                           file for conv values (octree_nn.npz) is absent from
                           the reference checkout, so no reference-held vector
                           pins conv values on sparse levels: for those the
                           pins are the ones above.
"""
