/*
 * C ABI of libcrystalformer_hip.so — MI355X (gfx950) kernels for Crystalformer's
 * infinitely connected attention.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller, float32 data,
 *     int64 indices, contiguous row-major tensors;
 *   - `stream` is a hipStream_t (NULL = the default stream); calls are
 *     asynchronous on it and never synchronise the device;
 *   - the library allocates nothing unless a function's comment says so;
 *   - return value 0 = success, negative = error (cf_last_error() gives the
 *     text for the calling thread); no kernel is launched on error;
 *   - optional pointers are documented as "nullable".
 *
 * Each entry point replaces one kernel launch of the reference's CuPy layer
 * (file:line under the reference checkout given per function).
 */
#ifndef CRYSTALFORMER_HIP_H
#define CRYSTALFORMER_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CF_OK 0
#define CF_ERR_INVALID_ARGUMENT (-1)
#define CF_ERR_UNSUPPORTED (-2)
#define CF_ERR_HIP (-3)

/* Library version, major*10000 + minor*100 + patch. */
int cf_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char *cf_last_error(void);

/* Largest translation half-width a rule-B box may take per axis; larger
 * values (or NaN exponents) are clamped so that a kernel always terminates. */
int cf_max_translation_range(void);

/*
 * Share of the GPU that one forward launch of the periodic encoding may occupy, for the
 * calling thread (default 1).  The forward pair kernel is persistent: it launches two
 * work-groups per CU, which hold the CU's whole register file, so kernels of other streams
 * wait for it to drain.  A caller that keeps several streams busy (several forwards in
 * flight) sets a share below 1: the kernel launches that fraction of its work-groups, runs
 * longer on its own, and leaves room beside it; results are bit-identical.  Read at launch
 * (a captured graph keeps the share it was captured with).  The backward kernel ignores
 * it.  No counterpart in the reference, whose launches are sized by the problem alone
 * (models/cuda_funcs/real_space_enc_proj.py:75-96).
 */
int cf_set_launch_share(double share);
double cf_get_launch_share(void);

/*
 * Batch sizes that only the device knows, for the calling thread.  For callers that replay ONE
 * captured graph (or keep one set of buffers) over batches whose crystal sizes differ: buffers
 * and launch grids are sized for capacities, and the live counts are read on the device.  No
 * counterpart in the reference, whose wrappers read the sizes back to the host on every call
 * (models/cuda_funcs/fused_dpa.py:73,137; models/cuda_funcs/irregular_mean.py:29-36).
 *
 *   header_4  DEVICE, four int64 words: live atoms N, live edges E, live atom pairs U, status.
 *             cf_batch_layout writes them from `sizes_n` as it finds it when its kernels run
 *             (status 1 and N = E = U = 0 when a size is negative or the totals exceed the
 *             capacities: every kernel below then does nothing).  NULL switches the mode off.
 *   N_cap, E_cap  the capacities; their sum must be even (U_cap = (N_cap + E_cap) / 2).
 * While a header is set, an entry point listed here that is called with N == N_cap (E == E_cap,
 * U == U_cap) takes that argument as the capacity -- array strides, launch grid -- and works on
 * the first live N (E, U) items only; results for those are bit-identical to a call with the
 * live sizes as arguments.  Entry points: cf_batch_layout, cf_edge_index, cf_edge_pairs,
 * cf_gauss_exponents, cf_linear_rows (rows = atoms), cf_real_enc_ring_stage,
 * cf_real_enc_fwd_rings (either rule), cf_real_enc_fwd (pair list; without one it refuses),
 * cf_fused_dpa_fwd.  The other
 * entry points ignore the header (per-crystal ones run over all B lattices handed in; crystals
 * beyond the live ones must have size 0).  Read at launch: a captured graph keeps the header
 * address it was captured with.
 */
int cf_set_size_header(int64_t *header_4, int64_t N_cap, int64_t E_cap);
const int64_t *cf_get_size_header(void);

/*
 * Real-space periodic encoding, forward.
 * Replaces the launches of real_enc_fwd / real_enc_proj_fwd
 * (models/cuda_funcs/real_space_enc.py:96-113,
 *  models/cuda_funcs/real_space_enc_proj.py:70-88;
 *  kernels models/kernels/real_enc_fwd.cu, real_enc_proj_fwd.cu).
 *
 *   a_ik      (N,H)    negative Gaussian exponents
 *   rpos_ij_e (E,3)    p_j - p_i per edge
 *   tvecs_n   (B,3,3)  lattice rows per crystal
 *   batch_i   (N)      crystal of each atom
 *   edge_ij_e (2,E)    edges (source i, target j)
 *   K         number of Gaussian value-PE bins, 0 = bias only (1..128 supported)
 *   D         rows of W (head dim of the projected value PE); ignored if W_k NULL
 *   W_k       nullable, (W_num,H,D,K); W_num in {1,E,N}
 *   rvlen_n   nullable, (B,3) lengths of the reciprocal lattice vectors
 *   cutoff_radius  0: fixed cube [-lattice_range,lattice_range]^3 (rule A);
 *                  <0: adaptive box from sqrt(-0.5/a)*|cutoff| per (atom,head);
 *                  >0: adaptive box from that radius.  Non-zero needs rvlen_n.
 *   minimum_range  lower bound of every adaptive half-width (0 = none)
 *   pairs_u   nullable, (U,5) unit descriptors as written by cf_edge_pairs: for
 *             every unordered pair of atoms of a crystal (self pairs included)
 *             the edge (i->j), i <= j, its reverse (j->i), the atoms i and j and
 *             the crystal.  When given (and K > 0) the two directions of a pair
 *             are evaluated together on the matrix cores; every edge must
 *             appear in exactly one descriptor and its reverse must carry
 *             rpos = -rpos.  NULL selects the per-edge kernels, which accept
 *             any edge list.
 *   sched_2   nullable, with pairs_u only: two int32 words holding 0.  With them the
 *             work-groups draw their rounds of units from a shared counter (they finish
 *             together whatever the units cost); without, rounds are dealt out in a fixed
 *             stride.  Results are identical bit for bit either way.  The words are 0 again
 *             when the launch completes and may serve the next launch on the same stream;
 *             launches that can overlap in time need words of their own.
 * Outputs
 *   z_ek  (E,H)                       log sum_n exp(a d^2)
 *   v_ekd nullable if K==0; (E,H,K) when W_k is NULL, else (E,H,D)
 */
int cf_real_enc_fwd(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                    const int64_t *batch_i, const int64_t *edge_ij_e,
                    int64_t N, int64_t H, int64_t E, int64_t B, int64_t K, int64_t D,
                    double dist_max, double wscale, const float *W_k, int64_t W_num,
                    const float *rvlen_n, double cutoff_radius, int lattice_range,
                    int minimum_range, const int64_t *pairs_u, int64_t U, int32_t *sched_2,
                    float *z_ek, float *v_ekd, void *stream);

/*
 * Staged translations kept across the blocks of a model (fixed cube, cutoff_radius = 0, of at
 * most 128 translations; K >= 1).  No counterpart in the reference, whose kernels redo the
 * geometry of every (edge, head, translation) in every block
 * (models/kernels/real_enc_proj_fwd.cu:94-131).
 *
 * What cf_real_enc_fwd stages per unit of pairs_u -- which translations reach a Gaussian bin, in
 * which order they are accumulated, their squared distance and Gaussian argument, the smallest
 * squared distance -- depends on rpos_ij_e, tvecs_n and the bin grid (K, dist_max, wscale) only,
 * not on a_ik.  cf_real_enc_ring_stage writes it once for all units into `rings`
 * (cf_real_enc_ring_bytes(U) bytes of device memory, 256-byte aligned); cf_real_enc_fwd_rings is
 * cf_real_enc_fwd (shared W_k of shape (H,D,K), D <= 32, pair list) starting from it.  The rings
 * stay valid while the positions, the lattices, the pair list and the bin grid do.
 *   weakest_exponent  upper bound (<= 0) of every a_ik the rings will be used with, e.g.
 *                     -gauss_lb / (2 r0^2): translations that reach no bin are kept only if
 *                     exp(weakest_exponent (d^2 - d^2_min)) > 2^-40.  Exponents above the bound
 *                     make the lattice sums drop terms they should hold; 0 keeps every translation.
 * Adaptive boxes (rvlen_n given and cutoff_radius != 0, the rule of
 * models/kernels/real_enc_fwd.cu:58-85): atom pairs whose (atom, head) half-widths all come out as
 * lattice_range have exactly the cube and are evaluated from the rings; the others are staged and
 * evaluated as cf_real_enc_fwd does.  Three launches: the range rule per atom pair (a byte per
 * pair, a count per chunk of 128); a stable partition of the pair indices into two lists, the
 * pairs that keep the cube first, with both lengths beside them; then one launch whose
 * work-groups take one of two roles, the rings' body over the first list and the staging body
 * over the second, the split worked out on the device from the two lengths (where fewer than
 * half the pairs keep the cube the staging body takes all of them).  All of it lives in `flags`:
 * cf_real_enc_flag_bytes(U, H) = 32 + 8 (ceil(U/2) + ceil(ceil(U/128)/2) + ceil(U/8)) bytes of
 * device scratch, 8-byte aligned, written and read by the call; nothing in it needs clearing.
 * The last launch needs up to 87 KB of dynamic LDS per work-group at K > 64 (53 KB at K <= 64).
 * More than 8 heads: the staging body alone, over all pairs.  Works under a size header (U is
 * then the capacity).  With the fixed cube rpos_ij_e, tvecs_n, batch_i, edge_ij_e, rvlen_n and
 * flags may be NULL, and there is one launch.
 */
int64_t cf_real_enc_ring_bytes(int64_t U);
int64_t cf_real_enc_flag_bytes(int64_t U, int64_t H);
int cf_real_enc_ring_stage(const float *rpos_ij_e, const float *tvecs_n, const int64_t *pairs_u, int64_t U,
                           int64_t K, double dist_max, double wscale, int lattice_range,
                           double weakest_exponent, void *rings, void *stream);
int cf_real_enc_fwd_rings(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                          const int64_t *batch_i, const int64_t *edge_ij_e, const int64_t *pairs_u,
                          int64_t U, int64_t N, int64_t H, int64_t E, int64_t K, int64_t D,
                          double dist_max, double wscale, const float *W_k, const float *rvlen_n,
                          double cutoff_radius, int lattice_range, int minimum_range,
                          const void *rings, void *flags, int64_t flag_bytes, float *z_ek,
                          float *v_ekd, void *stream);
/*
 * cf_real_enc_bwd (below; same arguments, workspace and results) for the fixed cube and one
 * projection per head, with the rings staged for this geometry, pair list, bin grid and
 * lattice_range: its pair kernel (K <= 64, D <= 16, gv_ekd given) starts from them; other shapes
 * run the kernels cf_real_enc_bwd runs, which do not read the rings.
 */
int cf_real_enc_bwd_rings(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                          const int64_t *batch_i, const int64_t *edge_ij_e, const int64_t *e_start_i,
                          const float *z_ek, const float *gz_ek, const float *gv_ekd,
                          int64_t N, int64_t H, int64_t E, int64_t B, int64_t K, int64_t D,
                          double dist_max, double wscale, const float *W_k, int lattice_range,
                          const int64_t *pairs_u, int64_t U, const float *rings, void *workspace,
                          int64_t workspace_bytes, float *ga_ik, float *gW_k, void *stream);

/*
 * Bytes of device scratch cf_real_enc_bwd needs for the given sizes
 * (pass want_gW != 0 when gW_k will be requested).
 */
int64_t cf_real_enc_bwd_workspace(int64_t N, int64_t H, int64_t E, int64_t K, int64_t D,
                                  int64_t W_num, int want_gW);

/*
 * Real-space periodic encoding, backward wrt a_ik and W_k.
 * Replaces the launches of real_enc_bwd / real_enc_proj_bwd
 * (models/cuda_funcs/real_space_enc.py:222-241,
 *  models/cuda_funcs/real_space_enc_proj.py:153-173;
 *  kernels models/kernels/real_enc_bwd.cu, real_enc_proj_bwd.cu).
 *
 *   e_start_i (N+1)  CSR offsets of each source atom's edges
 *   z_ek      (E,H)  forward output
 *   gz_ek     (E,H)  gradient of z
 *   gv_ekd    nullable; (E,H,K) when W_k is NULL else (E,H,D)
 *   workspace device scratch of cf_real_enc_bwd_workspace() bytes (256-byte aligned)
 *   pairs_u   nullable, (U,5) unit descriptors as for cf_real_enc_fwd; with it (and a shared
 *             W_k, K <= 64, D <= 16) the two directions of a pair are evaluated together
 *             on the matrix cores
 * Outputs
 *   ga_ik (N,H)
 *   gW_k  nullable; (W_num,H,D,K) — already reduced to W's own shape (the
 *         reference returns per-atom partial sums and lets autograd reduce them)
 */
int cf_real_enc_bwd(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                    const int64_t *batch_i, const int64_t *edge_ij_e,
                    const int64_t *e_start_i, const float *z_ek, const float *gz_ek,
                    const float *gv_ekd, int64_t N, int64_t H, int64_t E, int64_t B,
                    int64_t K, int64_t D, double dist_max, double wscale,
                    const float *W_k, int64_t W_num, const float *rvlen_n,
                    double cutoff_radius, int lattice_range, int minimum_range,
                    const int64_t *pairs_u, int64_t U,
                    void *workspace, int64_t workspace_bytes,
                    float *ga_ik, float *gW_k, void *stream);

/*
 * cf_real_enc_bwd without a workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference, whose wrappers allocate their scratch with
 * torch.empty on every call (models/cuda_funcs/real_space_enc_proj.py:137-151).
 *
 * Same arguments, kernels and results as cf_real_enc_bwd; the scratch lives in a fixed
 * array of cf_static_scratch_bytes() = 32 MiB inside the library's device code, which every
 * GPU the library runs on holds until the process ends.  Sizes for which
 * cf_real_enc_bwd_workspace() exceeds that are rejected with CF_ERR_INVALID_ARGUMENT (the
 * benchmark's training batch of 128 crystals needs 18.6 MB, 256 crystals of up to 96 atoms
 * 24 MB).  Calls nothing that allocates or frees.  All calls on one GPU share the one array:
 * calls that overlap in time on the same GPU (different streams or threads) race and give
 * wrong gradients; calls on one stream are ordered and safe.
 */
int64_t cf_static_scratch_bytes(void);
int cf_real_enc_bwd_static(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                           const int64_t *batch_i, const int64_t *edge_ij_e,
                           const int64_t *e_start_i, const float *z_ek, const float *gz_ek,
                           const float *gv_ekd, int64_t N, int64_t H, int64_t E, int64_t B,
                           int64_t K, int64_t D, double dist_max, double wscale,
                           const float *W_k, int64_t W_num, const float *rvlen_n,
                           double cutoff_radius, int lattice_range, int minimum_range,
                           const int64_t *pairs_u, int64_t U,
                           float *ga_ik, float *gW_k, void *stream);

/*
 * Lattice-sum bias and the attention that consumes it in one launch, for blocks without
 * Gaussian value bins (K = 0, the "simplified" model): out[i,h,:] = sum_j softmax_j(q_i.k_j +
 * z_ij)[j] v_j with z_ij = log sum_n exp(a_ih |r_ij + n.L|^2), z and the probabilities kept
 * on chip.  Replaces the pair of launches real_enc_proj_fwd -> fused_dpa_fwd
 * (models/cuda_funcs/real_space_enc_proj.py:70-97 followed by
 *  models/cuda_funcs/fused_dpa.py:36-61) when nothing downstream needs z (inference).
 *
 * Arguments as for cf_real_enc_fwd (K = 0) and cf_fused_dpa_fwd (no b_ij); que is pre-divided
 * by sqrt(Dk).  edge_ij_e must be sorted by source atom (e_start_i its CSR offsets); any
 * such list is accepted.  max_row is a HARD upper bound on the edges of one source atom: a
 * work-group keeps its row's max_row * H logits in LDS, 64 KB at most (rows of up to 1820
 * edges at H = 8), beyond that CF_ERR_UNSUPPORTED.  The host cannot check the bound against
 * e_start_i without reading it back; a row that exceeds it is not evaluated and its output row
 * is NaN.
 * Output: out (N,H,Dv); rows of atoms without edges are zero.
 */
int cf_fused_enc_dpa_fwd(const float *a_ik, const float *rpos_ij_e, const float *tvecs_n,
                         const int64_t *batch_i, const int64_t *edge_ij_e, const int64_t *e_start_i,
                         const float *que, const float *key, const float *val,
                         int64_t N, int64_t H, int64_t E, int64_t B, int64_t Dk, int64_t Dv,
                         const float *rvlen_n, double cutoff_radius, int lattice_range,
                         int minimum_range, int64_t max_row, float *out, void *stream);

/*
 * Per (atom, head) translation half-widths the encoding kernels use,
 * R_out (N,H,3) int32.  Exposes the rule of models/kernels/real_enc_fwd.cu:58-85
 * for bit-exact checks and work counting.
 */
int cf_translation_ranges(const float *a_ik, const float *rvlen_n, const int64_t *batch_i,
                          int64_t N, int64_t H, double cutoff_radius, int lattice_range,
                          int minimum_range, int32_t *R_out, void *stream);

/*
 * Fused edge-indexed dot-product attention, forward.
 * Replaces the launch of fused_dpa_fwd / fused_dpa_fwd_v3
 * (models/cuda_funcs/fused_dpa.py:40-57; kernel models/kernels/fused_dpa_fwd.cu).
 * No limit on atoms per crystal.
 *
 *   que (N,H,Dk) already divided by sqrt(Dk); key (N,H,Dk); val (N,H,Dv)
 *   aij_eh  nullable (E,H) additive logit bias
 *   bij_ehd nullable (E,H,Dv) additive value term
 *   edge_ij_e (2,E) sorted by source atom; e_start_i (N+1) CSR offsets
 * Outputs
 *   prob_eh (E,H) softmax over each source atom's edges
 *   out     (N,H,Dv)
 */
int cf_fused_dpa_fwd(const float *que, const float *key, const float *val,
                     const float *aij_eh, const float *bij_ehd, const int64_t *edge_ij_e,
                     const int64_t *e_start_i, int64_t N, int64_t H, int64_t E,
                     int64_t Dk, int64_t Dv, float *prob_eh, float *out, void *stream);

/*
 * Fused attention, backward.  Replaces irregular_transpose + fused_dpa_bwd +
 * fused_dpa_bwd_q (models/cuda_funcs/fused_dpa.py:141-206; kernels
 * models/kernels/fused_dpa_bwd.cu, fused_dpa_bwd_q.cu, irregular_transpose.cu).
 * The edge list must be the dense per-crystal block layout produced by
 * cf_edge_index (edge of (i,j) in a crystal of n atoms at e0 + i*n + j): the
 * key-side sums walk a column of that block instead of transposing it.
 *
 *   batch_i (N); atom_start_n (B+1) first atom of each crystal;
 *   edge_start_n (B+1) first edge of each crystal
 *   prob_eh, out: forward outputs; gout (N,H,Dv)
 * Outputs
 *   gque (N,H,Dk) (gradient wrt the pre-scaled query), gkey, gval,
 *   gaij (E,H), gbij nullable (E,H,Dv)
 */
int cf_fused_dpa_bwd(const float *que, const float *key, const float *val,
                     const float *bij_ehd, const int64_t *batch_i,
                     const int64_t *edge_ij_e, const int64_t *e_start_i,
                     const int64_t *atom_start_n, const int64_t *edge_start_n,
                     int64_t N, int64_t H, int64_t E, int64_t B, int64_t Dk, int64_t Dv,
                     const float *prob_eh, const float *out, const float *gout,
                     float *gque, float *gkey, float *gval, float *gaij, float *gbij,
                     void *stream);

/*
 * Per-crystal mean over atoms.  Replaces the launch of irregular_mean_fwd
 * (models/cuda_funcs/irregular_mean.py:43-54; kernel
 * models/kernels/irregular_mean_fwd.cu).  No limit on atoms per crystal.
 *   src (N,D); start_n (B+1) -> dst (B,D)
 */
int cf_irregular_mean_fwd(const float *src, const int64_t *start_n, int64_t B, int64_t D,
                          float *dst, void *stream);

/* Backward of the mean: gx[i,:] = go[batch_i[i],:] / len(batch_i[i])
 * (models/cuda_funcs/irregular_mean.py:60-69). */
int cf_irregular_mean_bwd(const float *go, const int64_t *batch_i, const int64_t *start_n,
                          int64_t N, int64_t D, float *gx, void *stream);

/*
 * Per-edge minimum squared distance over the translation box.  Replaces the
 * launch of minimum_distance (models/cuda_funcs/minimum_distance.py:30-40;
 * kernel models/kernels/minimum_distance.cu).
 */
int cf_minimum_distance(const float *rpos_ij_e, const float *tvecs_n, const int64_t *batch_i,
                        const int64_t *edge_ij_e, int64_t E, const float *rvlen_n,
                        double cutoff_radius, int lattice_range, int minimum_range,
                        float *dist2_min_e, void *stream);

/*
 * Dense intra-crystal edge list and relative positions on the device.
 * Replaces the host loops of get_edge_index and the pos[j]-pos[i] gather
 * (models/indexed_latticeformer_encoder.py:15-32, 214).
 *   atom_start_n, edge_start_n (B+1): leading-zero cumulative sums of sizes
 *   and sizes^2;  pos (N,3) nullable (then rpos_ij_e is not written)
 * Outputs
 *   edge_ij_e (2,E), nullable when only the relative positions of a known
 *   layout are wanted; rpos_ij_e nullable (E,3)
 */
int cf_edge_index(const int64_t *atom_start_n, const int64_t *edge_start_n, int64_t B,
                  int64_t E, const float *pos, int64_t *edge_ij_e, float *rpos_ij_e,
                  void *stream);

/*
 * Unit descriptors of the dense per-crystal edge blocks: for each crystal of n
 * atoms the n(n+1)/2 pairs (i <= j) in row-major order of the upper triangle,
 * five words each: edge (i->j), edge (j->i), atom i, atom j, crystal.
 * No counterpart in the reference (its kernels treat the two directions of an
 * edge independently, models/kernels/real_enc_proj_fwd.cu:24-31).
 *   atom_start_n, edge_start_n, unit_start_n (B+1): leading-zero cumulative
 *   sums of sizes, sizes^2 and sizes*(sizes+1)/2
 * Output
 *   pairs_u (U,5) with U = unit_start_n[B] = (E + N) / 2
 */
int cf_edge_pairs(const int64_t *atom_start_n, const int64_t *edge_start_n,
                  const int64_t *unit_start_n, int64_t B, int64_t E, int64_t *pairs_u,
                  void *stream);

/*
 * Cell volume, reciprocal lattice vectors and their lengths, one launch:
 *   vcell_n = det(trans_n)            (term order of models/indexed_latticeformer_encoder.py:34-44)
 *   recip_n = 2 pi (a2 x a3, a3 x a1, a1 x a2) / vcell_n      (models/indexed_latticeformer_encoder.py:206-212)
 *   rvlen_n = row norms of recip_n    (models/indexed_lattice_multi_head_attention_cuda.py:879, torch.norm)
 * Replaces the ~25 elementwise launches those expressions take.
 *   trans_n (B,3,3); outputs vcell_n (B), recip_n (B,3,3), rvlen_n (B,3), each nullable.
 */
int cf_lattice_geometry(const float *trans_n, int64_t B, float *vcell_n, float *recip_n,
                        float *rvlen_n, void *stream);

/*
 * Gaussian exponents of the periodic encoding from the per-head query
 * (models/indexed_lattice_multi_head_attention_cuda.py:636-722, gauss_state "q"):
 *   alpha[i,h] = sum_d q[i,h,d] w[h,d]
 *   normalize:  alpha = (alpha + shift) * scale, with (scale, shift) =
 *               gauss_scale when gauss_scale[0] > 0, else (1/std, -mean) of
 *               alpha over the whole batch (unbiased std); update_stats
 *               stores the pair used back into gauss_scale
 *   a[i,h]     = coef * rho(alpha),   coef = -1 / (2 r0^2)
 *   rho        : 0 elu  (1-lb) elu(x beta/(1-lb)) + 1
 *                1 abs  (1-lb) |x| + lb
 *                2 exp  (1-lb) exp(x beta/(1-lb)) + lb
 *                (models/indexed_lattice_multi_head_attention_cuda.py:675-692)
 *   q_scaled   = q * q_scale (nullable), the query the attention consumes
 *   alpha_n    = normalised alpha (nullable), what a backward pass needs
 * Replaces ~14 elementwise / reduction launches per attention block.  Two
 * launches, fixed summation order.
 *   workspace: cf_gauss_exponents_workspace(N,H) bytes when normalize != 0; on
 *              return floats [-4], [-3] of it hold the (scale, shift) pair used
 */
int64_t cf_gauss_exponents_workspace(int64_t N, int64_t H);
int cf_gauss_exponents(const float *q_ihd, const float *w_hd, float *gauss_scale, int64_t N, int64_t H,
                       int64_t D, int normalize, int update_stats, int positive_func, float beta,
                       float lower_bound, float coef, float q_scale, void *workspace,
                       int64_t workspace_bytes, float *alpha_n, float *a_ih, float *q_scaled,
                       void *stream);

/*
 * Backward of cf_gauss_exponents with the normalisation statistics held constant (the
 * reference detaches them, models/indexed_lattice_multi_head_attention_cuda.py:700-712; what
 * autograd computes for :636-722): g_alpha = ga * rho'(alpha_n) * coef * scale,
 * gq = g_alpha w_head + gqs * q_scale, gw[h] = sum_i g_alpha[i,h] q[i,h] in a fixed order.
 *   ga (N,H) or NULL (no gradient through a), gqs (N,H,D) or NULL, alpha_n (N,H) as left by the
 *   forward, used_scale: DEVICE pointer to the scale the forward applied, NULL when it did
 *   not normalise; gq (N,H,D) and gw (H,D): either may be NULL
 *   workspace: cf_gauss_exponents_bwd_workspace(N,H,D) bytes, needed when gw is asked for
 */
int64_t cf_gauss_exponents_bwd_workspace(int64_t N, int64_t H, int64_t D);
int cf_gauss_exponents_bwd(const float *ga, const float *gqs, const float *q, const float *w,
                           const float *alpha_n, const float *used_scale, int64_t N, int64_t H, int64_t D,
                           int positive_func, float beta, float lower_bound, float coef, float q_scale,
                           void *workspace, int64_t workspace_bytes, float *gq, float *gw, void *stream);

/*
 * Row-block linear layer(s): y_w = act(x W_w^T + b_w) (+ residual), w < n_weights <= 3,
 * for the small dense layers around the attention: the query/key/value
 * projections in one launch (models/indexed_lattice_multi_head_attention_cuda.py:865-867,
 * three F.linear calls), the output projection with its residual and the two
 * feed-forward layers with ReLU / residual fused
 * (models/indexed_latticeformer_encoder.py:806-826, F.linear + activation + add).
 * fp32 on the matrix cores; inference path (no autograd).
 *   x (N,K), K a multiple of 16;  w0..w2 each (C,K) row-major;  bias (n_weights*C) nullable
 *   residual (N,C) nullable, only with n_weights == 1;  relu != 0 applies max(.,0) last
 * Outputs
 *   y0..y2 each (N,C)
 */
int cf_linear_rows(const float *x, int64_t N, int64_t K, const float *w0, const float *w1,
                   const float *w2, int n_weights, int64_t C, const float *bias,
                   const float *residual, int relu, float *y0, float *y1, float *y2, void *stream);

/*
 * Input gradient of linear layers (what autograd computes for the F.linear calls cited at
 * cf_linear_rows): y (N,K) = mask(sum_i g_i W_i) + add, g_i (N,C), W_i (C,K) row-major, 1..3 terms
 * of equal shapes (query / key / value projections share their input); add (N,K) or NULL (a
 * gradient arriving on a residual branch); mask (N,K) or NULL: where mask <= 0 the product is
 * zeroed (the ReLU in front of the layer).  C a multiple of 64, K of 4.
 */
int cf_linear_rows_nn(const float *g0, const float *g1, const float *g2, int n_terms, const float *w0,
                      const float *w1, const float *w2, int64_t N, int64_t C, int64_t K, const float *add,
                      const float *mask, float *y, void *stream);

/*
 * Column sums of a row-major (N,C) matrix, out (C): the bias gradient of the linear layers
 * (what autograd computes for the F.linear calls cited at cf_linear_rows), in a fixed
 * order, one launch, no scratch.
 */
int cf_column_sum(const float *g, int64_t N, int64_t C, float *out, void *stream);

/*
 * Weight gradient of a linear layer, gW (C,K) = g^T x for g (N,C), x (N,K) (what autograd
 * computes for the F.linear calls cited at cf_linear_rows): rows cut into slices summed in a
 * fixed order, fp32 on the matrix cores.  gb (C) or NULL: the bias gradient (column sums of
 * g) from the same pass over g.
 *   workspace: cf_linear_weight_grad_workspace(N,C,K) bytes
 */
int64_t cf_linear_weight_grad_workspace(int64_t N, int64_t C, int64_t K);
int cf_linear_weight_grad(const float *g, const float *x, int64_t N, int64_t C, int64_t K,
                          void *workspace, int64_t workspace_bytes, float *gW, float *gb, void *stream);

/*
 * Reciprocal-space periodic encoding (ReciPeriodicEncodingFuncCUDA, models/cuda_funcs/reci_space_enc.py:17-99;
 * kernels models/kernels/reci_enc_fwd.cu:3-68, reci_enc_bwd.cu:3-71), LATTICE_RANGE passed at run time:
 *   S[e,h] = sum over n1 in [0,R] (weight 2 for n1 != 0), n2, n3 in [-R,R] of
 *            exp(a[i,h] |n1 b1 + n2 b2 + n3 b3|^2) cos(<kr_base[e], n>),  b_d = rows of rvecs_n[batch[i]]
 *   z[e,h] = log(max(S, 1e-6)) + 1.5 log(-4 pi a[i,h]) - log(vcell_n[batch[i]]),  sumexp[e,h] = S
 *   ga[i,h] = sum over the edges e of row i of gz[e,h] / S[e,h] * dS/da (0 where S < 1e-6); with
 *            normalisation_grad == 0 as the reference's kernel, which leaves out the derivative
 *            of the 1.5 log(-4 pi a) term; != 0 adds it (1.5 / a[i,h] * sum_e gz[e,h]), which is
 *            what autograd gives on the reference's PyTorch path.
 * Edges are addressed through their row offsets e_start_i (N+1) (edges sorted by source atom, as
 * the reference's backward assumes, reci_space_enc.py:66-68); kr_base_e (E,3) are the phases
 * <b_d, p_j - p_i> (models/indexed_latticeformer_encoder.py:245-251), which cf_kr_base computes.
 * Limits: H <= 16, (R+1)(2R+1)^2 * padded H <= 8192.
 */
int cf_kr_base(const float *rpos_ij_e, const float *rvecs_n, const int64_t *batch_i, const int64_t *edge_ij_e,
               int64_t E, float *kr_base_e, void *stream);
int cf_reci_enc_fwd(const float *a_ik, const float *kr_base_e, const float *rvecs_n, const float *vcell_n,
                    const int64_t *batch_i, const int64_t *e_start_i, int64_t N, int64_t H, int64_t E,
                    int lattice_range, float *z_ek, float *sumexp_ek, void *stream);
int cf_reci_enc_bwd(const float *a_ik, const float *kr_base_e, const float *rvecs_n, const int64_t *batch_i,
                    const int64_t *e_start_i, const float *gz_ek, const float *sumexp_ek, int64_t N, int64_t H,
                    int64_t E, int lattice_range, int normalisation_grad, float *ga_ik, void *stream);

/*
 * cf_linear_weight_grad for n_layers linear layers at once (2 * ceil(n_layers / 32)
 * launches instead of 2 * n_layers); per layer the result is bit-identical to the single
 * call.  g, x, gW, gb: HOST arrays of device pointers (gb[t] may be NULL); N, C, K: HOST
 * arrays.  workspace: cf_linear_weight_grad_grouped_workspace(n_layers, N, C, K) bytes.
 */
int64_t cf_linear_weight_grad_grouped_workspace(int n_layers, const int64_t *N, const int64_t *C,
                                                const int64_t *K);
int cf_linear_weight_grad_grouped(int n_layers, const float *const *g, const float *const *x, const int64_t *N,
                                  const int64_t *C, const int64_t *K, float *const *gW, float *const *gb,
                                  void *workspace, int64_t workspace_bytes, void *stream);

/*
 * One optimiser update of a training step over n_tensors parameter tensors: global
 * gradient-norm clip (nn.utils.clip_grad_norm_, models/regression.py:122), AdamW
 * (optim.AdamW, models/regression.py:254; decoupled weight decay per tensor, betas, eps)
 * and the schedule lr0 * sqrt(sch_decay / (sch_decay + t)) of models/regression.py:269
 * (sch_decay <= 0: constant lr0), in 2 * ceil(n_tensors / 64) launches.
 *   params, grads, exp_avg, exp_avg_sq: HOST arrays of n_tensors device pointers (read at
 *       call time and passed to the kernels by value; the device memory they name is read
 *       and written when the kernels run)
 *   numel, weight_decay: HOST arrays of n_tensors element counts / decay factors
 *   clip_norm <= 0: no clipping
 *   state_3: DEVICE, [0] updates taken so far, counted in fp32 (exact below 2^24; zero it
 *       once; every call adds one before using it), [1] gradient norm of this call,
 *       [2] learning rate of this call
 *   workspace: cf_adamw_step_workspace(n_tensors, numel) bytes (DEVICE)
 */
int64_t cf_adamw_step_workspace(int n_tensors, const int64_t *numel);
int cf_adamw_step(int n_tensors, float *const *params, const float *const *grads, float *const *exp_avg,
                  float *const *exp_avg_sq, const int64_t *numel, const float *weight_decay, float lr0,
                  float sch_decay, float beta1, float beta2, float eps, float clip_norm, float *state_3,
                  void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Every index structure of a batch of crystals with dense intra-crystal edges from the crystal
 * sizes, in four launches and without a host round trip: what get_edge_index
 * (models/indexed_latticeformer_encoder.py:15-32), the CSR offsets of
 * models/cuda_funcs/fused_dpa.py:24-26 and cf_edge_pairs compute one by one.
 *   sizes_n (B) atoms per crystal; N = sum n, E = sum n^2 (the caller knows them: it sized
 *   the outputs)
 * Outputs
 *   atom_start_n, edge_start_n, unit_start_n (B+1): leading-zero cumulative sums of n, n^2,
 *       n (n + 1) / 2
 *   e_start_i (N+1), edge_ij_e (2,E), pairs_u ((E+N)/2, 5) or NULL
 *   batch_i (N) or NULL: crystal of each atom, numbered from 0 (what the data loader's `batch`
 *       holds after the rebasing of models/indexed_latticeformer_encoder.py:436,722)
 * With a size header set for (N, E) (cf_set_size_header) N and E are capacities, `sizes_n` may hold
 * zeros past the live crystals, and the header is written here.
 */
int cf_batch_layout(const int64_t *sizes_n, int64_t B, int64_t N, int64_t E, int64_t *atom_start_n,
                    int64_t *edge_start_n, int64_t *unit_start_n, int64_t *e_start_i, int64_t *edge_ij_e,
                    int64_t *pairs_u, int64_t *batch_i, void *stream);

/*
 * Up to 8 device-to-device copies in one launch: dst[s][0..bytes[s]) = src[s][0..bytes[s]), or
 * zeros where src[s] is NULL.  src, dst, bytes: HOST arrays of n_segments entries (device
 * addresses, read at call time and passed to the kernel by value).  Segments must not overlap.
 * For a caller that refreshes the input buffers of a captured graph with a new batch (features,
 * positions, lattices, sizes): one launch instead of one per tensor.  No counterpart in the
 * reference, which hands every batch to its kernels in the loader's own tensors.
 */
int cf_copy_segments(int n_segments, const void *const *src, void *const *dst, const int64_t *bytes,
                     void *stream);

/*
 * Training loss of the regression module and its gradient in one launch: the per-sample
 * L1 losses summed over the targets (losses/regression_loss.py:10-20 with loss_fn "l1"),
 * averaged over the batch (models/regression.py:117-118).
 *   pred, target: (B, T) row-major; loss: (1); grad: (B, T) = sign(pred - target) / B, or NULL
 * One work-group, fixed summation order.
 */
int cf_l1_mean_loss(const float *pred, const float *target, int64_t B, int64_t T, float *loss, float *grad,
                    void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CRYSTALFORMER_HIP_H */
