// The entry points of hordead_gpu.h as a table of function pointers.
#include "hordead_gpu.h"

extern "C" const hgpu_api* hgpu_get_api(void) {
  static const hgpu_api api = {
      sizeof(hgpu_api),
      hgpu_init,        hgpu_shutdown,  hgpu_sync,        hgpu_last_error, hgpu_upload,      hgpu_download,
      hgpu_read_scalar, hgpu_retain,    hgpu_release,     hgpu_rank,       hgpu_dtype_of,    hgpu_size,
      hgpu_shape,       hgpu_strides,   hgpu_is_dense,    hgpu_transpose,  hgpu_reshape,     hgpu_slice,
      hgpu_reverse,     hgpu_replicate, hgpu_index_prefix, hgpu_as_strided, hgpu_materialize, hgpu_pad,
      hgpu_ewise1,      hgpu_ewise2,    hgpu_compare,     hgpu_compare_all, hgpu_select,     hgpu_convert,
      hgpu_contract,    hgpu_argminmax_last, hgpu_iota,   hgpu_concat,     hgpu_gather,      hgpu_scatter_add,
      hgpu_onehot,      hgpu_fused_map, hgpu_scatter_affine,
      hgpu_capture_begin, hgpu_capture_end, hgpu_graph_launch, hgpu_graph_destroy, hgpu_overwrite, hgpu_contract_sum, hgpu_assign, hgpu_extremum_last, hgpu_fused_extremum, hgpu_fused_sum,
      hgpu_contract_map, hgpu_contract_operands, hgpu_fused_map_sums, hgpu_contract_sum_map, hgpu_fused_map_dimsum,
  };
  return &api;
}
