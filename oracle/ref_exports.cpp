// C-linkage trampolines appended to the reference's CPU functions when oracle/_ref/libref_cpu.so is built
// (see oracle/Makefile).  They add nothing but a stable symbol name for ctypes.
extern "C" {
void ref_attention_forward_cpu(float* Q, float* K, float* V, float softmax_scale, int batch_size, int n_heads,
                               int seq_len, int head_dim, float* output, int use_causal_mask, int window_size,
                               float* alibi_slopes)
{
    attention_forward_cpu(Q, K, V, softmax_scale, batch_size, n_heads, seq_len, head_dim, output,
                          use_causal_mask != 0, window_size, alibi_slopes);
}
int ref_num_splits_heuristic(int batch_nheads_mblocks, int num_SMs, int num_n_blocks, int max_splits, int seq_len)
{
    return num_splits_heuristic(batch_nheads_mblocks, num_SMs, num_n_blocks, max_splits, seq_len);
}
void ref_verfiy(float* O, float* O_host, int batch_size, int n_heads, int seq_len, int head_dim, float range_of_error)
{
    verfiy(O, O_host, batch_size, n_heads, seq_len, head_dim, range_of_error);
}
}
