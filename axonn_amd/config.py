"""Grid configuration globals, as axonn/config.py:7-10 plus the attributes
axonn/axonn.py:51-64 sets.  One GPU: every degree is 1 and every rank is 0."""

G_inter = 1
G_data = 1
G_intra = 1
G_intra_r = 1
G_intra_c = 1
G_intra_d = 1
inter_layer_parallel_rank = 0
data_parallel_rank = 0
intra_layer_parallel_rank = 0
intra_layer_depth_parallel_rank = 0
intra_layer_row_parallel_rank = 0
intra_layer_column_parallel_rank = 0
micro_batch_size = None
batch_size = None
batch_size_per_gpu = None
