"""MI355X (gfx950) implementation of the HGCalML custom-op hot path.

Public API (same names and signatures as the reference's Python wrappers):
BinByCoordinates, BinnedSelectKnn, IndexReplacer, AccumulateKnn,
AccumulateLinKnn, AccumulateKnnSumw, AccumulateLinKnnSumw, PushKnn,
BuildAndAssignCondensatesBinned, LocalDistance, NeighbourCovariance and the RaggedGravNet layer on top of them. All of them need tensors on
a HIP device and the in-tree libhgcalml_amd.so; there is no CPU path.
"""
__all__ = ["BinByCoordinates", "BinnedSelectKnn", "IndexReplacer", "AccumulateKnn", "AccumulateLinKnn",
           "AccumulateKnnSumw", "AccumulateLinKnnSumw", "PushKnn", "BuildAndAssignCondensatesBinned", "RaggedGravNet",
           "LocalDistance", "NeighbourCovariance"]


def __getattr__(name):
    # lazy: importing the package alone (e.g. for the build script) must not require the compiled library
    if name in __all__:
        import importlib
        mod = {
            "BinByCoordinates": "bin_by_coordinates_op",
            "BinnedSelectKnn": "binned_select_knn_op",
            "IndexReplacer": "index_replacer_op",
            "AccumulateKnn": "accknn_op",
            "AccumulateLinKnn": "accknn_op",
            "AccumulateKnnSumw": "accknn_op",
            "AccumulateLinKnnSumw": "accknn_op",
            "PushKnn": "push_knn_op",
            "RaggedGravNet": "GravNetLayersRagged",
            "LocalDistance": "local_distance_op",
            "NeighbourCovariance": "neighbour_covariance_op",
            "BuildAndAssignCondensatesBinned": "assign_condensate_op",
        }[name]
        return getattr(importlib.import_module("." + mod, __name__), name)
    raise AttributeError(name)
