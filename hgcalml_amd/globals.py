"""Module-level switches with the names of the reference's modules/globals.py:91-92.
When set, the wrappers use plain torch compositions (differentiable by autograd)
instead of the custom kernels."""
knn_ops_use_tf_gradients = False
acc_ops_use_tf_gradients = False
