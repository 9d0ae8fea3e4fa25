"""Run-time switches of the host wrappers."""

# Read the device status word after each kNN call and raise on non-finite input
# (one host synchronisation per call, as the reference's own checks do).  Set to
# False inside latency-critical loops that validate their inputs elsewhere.
sync_checks = True

# Accumulate the kNN kernel's counters (distance evaluations, candidate chunks,
# pool prunes) into binned_select_knn.last_stats; used by the benchmark.  Calls that collect them run the
# statistics build of the search kernels, which is slower (counters in the inner loops, one atomic per wavefront).
collect_stats = False

# When binned_select_knn is called without n_bins, size the search grid for this library's search (coarse bins
# over up to four dimensions) instead of with the reference's heuristic and max_bin_dims.  The neighbours
# returned are the same either way; only the run time differs.
auto_grid = True

# GravNetOp's backward: combine the feature gradients of 32 rows that are consecutive in the search's sorted order
# on chip before they are added to memory (K <= 64, 8 < P <= 64).  False: one atomic row update per (point, slot)
# pair, the kernel the stand-alone gravnet_aggregate op uses.  Same gradients up to float summation order.
tile_aggregation_backward = True

# binned_select_knn returns a row's neighbours (slots 1.., after the query itself in slot 0) in no particular order,
# as the reference does (its kernel replaces the farthest entry in place; its tests sort each row before comparing).
# True: by increasing distance, at the price of a per-query sort inside the search kernel (+10 % at 1 M points, K = 64).
# The neighbour set, the distances and the gradients are the same either way.
sorted_neighbours = False

# Searches over points with 5 to 8 coordinates (K <= 256, events of at most 65535 points) can screen their candidates
# on the matrix cores and compute exact distances only for the pairs that can still matter.  True: the library decides
# by the event sizes (where bounding boxes thin the candidates out well the vector-unit search is faster); False:
# always the vector-unit search; "always": the matrix cores wherever that search can run.  Same neighbours and
# bit-identical distances either way.
matrix_search = True
