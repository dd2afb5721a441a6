/*
 * libfastlstm_hip.so -- C ABI of the MI355X (gfx950) LSTM forward/backward path.
 *
 * The reference (oleicht/FastLSTM) is pure Python and has no FFI of its own:
 * its boundary for this path is the set of host functions in fastlstm/lstm.py
 * that launch Triton kernels and cuBLAS GEMMs.  Each entry point below replaces
 * one of those launch sites; the Python wrappers in fastlstm_amd/lstm.py bind
 * them with ctypes and keep the reference's Python signatures.
 *
 * Conventions
 *  - every data pointer is a DEVICE pointer owned by the caller, 16-byte
 *    aligned, densely packed row-major with the shapes given below;
 *  - `stream` is a hipStream_t passed as void*; every launch is asynchronous
 *    on it and nothing here synchronises the host;
 *  - the library never allocates device memory: scratch comes in through the
 *    `ws` arguments, sized by the *_workspace_bytes / plan calls; the leading part of a
 *    recurrence workspace (header, barrier counters, flags: plan->ws_zero_bytes) must be
 *    ZERO-FILLED by the caller before each call (the same contract as the reference's
 *    zero-initialised sync buffer, fastlstm/lstm.py:96-100, 249) -- see
 *    fastlstm_recurrent_workspace_bytes;
 *  - return value: 0 on success, a negative fastlstm_status otherwise; argument
 *    validation happens before the first HIP call, so the error paths can be
 *    exercised on a machine without a GPU;
 *  - dtype: element type of all activations/weights (fastlstm_dtype); all
 *    accumulation is fp32.
 */
#ifndef FASTLSTM_HIP_H
#define FASTLSTM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { FASTLSTM_FP32 = 0, FASTLSTM_FP16 = 1, FASTLSTM_BF16 = 2 } fastlstm_dtype;

typedef enum {
    FASTLSTM_OK = 0,
    FASTLSTM_ERR_NULL = -1,      /* a required pointer is NULL */
    FASTLSTM_ERR_DIM = -2,       /* non-positive or overflowing dimension */
    FASTLSTM_ERR_DTYPE = -3,     /* dtype not in fastlstm_dtype */
    FASTLSTM_ERR_ALIGN = -4,     /* pointer not 16-byte aligned */
    FASTLSTM_ERR_RESIDENCY = -5, /* the barrier group cannot be co-resident (H > 64 units x compute units) */
    FASTLSTM_ERR_WORKSPACE = -6, /* workspace smaller than required */
    FASTLSTM_ERR_HIP = -7,       /* a HIP runtime call failed (no device, launch error) */
    FASTLSTM_ERR_TIMEOUT = -8    /* a workspace status word reports a barrier time-out */
} fastlstm_status;

/* Tiling of one recurrent launch.  A workgroup owns `bt` batch rows x `ht`
 * hidden units (x 4 gates); the `n_htiles` workgroups of one batch tile
 * exchange h_t (forward) / d_ifgo_t (backward) every timestep and never talk
 * to other batch tiles.  n_btiles * n_htiles <= num_cus so that every
 * workgroup is resident while its peers spin (the rule of
 * fastlstm/configs.py:29-58); a batch that does not fit is processed in
 * `batch_chunks` sequential launches (fastlstm/kernels.py:514, 663).
 * The rule counts one launch at a time.  Two recurrent launches on different
 * streams of one GPU could each hold a part of the compute units and wait for
 * the other's missing workgroups until the time-out, so the library orders
 * them itself: every recurrent entry point records an event (one per device)
 * behind its launches, and the next recurrent entry point on ANOTHER stream of
 * that device makes its stream wait for that event first (hipStreamWaitEvent,
 * no host synchronisation).  Recurrent work of different streams therefore
 * runs one call after the other on a device.  Not covered: launches recorded
 * into a graph by stream capture (the library neither records nor waits while
 * a stream is capturing) -- replaying two such graphs at the same time, or one
 * next to an eager call, is for the caller to order. */
typedef struct {
    int num_cus;      /* compute units used for planning */
    int lds_limit;    /* bytes of LDS one workgroup may use */
    int bt, ht;       /* batch rows / hidden units per workgroup */
    int n_btiles;     /* batch tiles per launch */
    int n_htiles;     /* hidden tiles (= barrier group size); 1 => no cross-CU sync */
    int batch_chunks; /* sequential launches needed to cover B */
    int wave_split;   /* 0: waves split K, 1: waves split batch tiles, 2: waves split W rows (H <= 64, no cross-CU sync),
                         3: W_h does not fit on chip -- waves split K and the weight slice is streamed every step */
    int lds_bytes;    /* LDS the kernel will request */
    size_t ws_bytes;  /* smallest workspace the recurrent call accepts (2 exchange slots; wave_split 3: plus W_h once
                         in operand order, which the call itself writes) */
    size_t ws_zero_bytes; /* leading bytes of the workspace that must be zero (header + counters + flags) */
    int ring_needs_zero;  /* 1: B or H leave padding in the exchange blocks -> zero the whole workspace */
} fastlstm_plan;

/* Pure host function (no HIP call): the tiling rule for a device with
 * `num_cus` compute units and `lds_limit` bytes of LDS per workgroup.
 * backward = 0 plans fastlstm_fwd_persistent, 1 plans fastlstm_bwd_persistent.
 * Replaces fastlstm/configs.py:29-58, 146-276 (grid sizing + tile pruning). */
int fastlstm_plan_for(int num_cus, int lds_limit, int B, int H, int dtype, int backward,
                      fastlstm_plan *plan);

/* Same, for HIP device `device` (-1: the current one; queries CU count and LDS size).  The first
 * call for a device also probes, with one tiny kernel and a device synchronisation, whether the
 * workgroups of a launch are dealt to the 8 XCDs in turn; the XCD-local recurrent kernels are only
 * used on a device where that was seen.  The launch calls below never synchronise. */
int fastlstm_plan_device(int device, int B, int H, int dtype, int backward, fastlstm_plan *plan);

/* Workspace of a recurrent call for this plan: header, barrier counters, flags and TWO exchange slots in the
 * layout of whichever kernel family the call may choose (fastlstm_recurrent_kernel_kind) -- a few hundred KiB,
 * independent of T (h_t / d_ifgo[t] of step t live in slot t % 2; plans that stream W_h add one packed copy of
 * it).  At least plan->ws_bytes.  The first plan->ws_zero_bytes bytes must be zero; the rest only if
 * plan->ring_needs_zero. */
size_t fastlstm_recurrent_workspace_bytes(const fastlstm_plan *plan, int T, int H, int dtype, int backward);

/* K1 -- ifgo[T*B,4H] = x[T*B,I] . Wx[4H,I]^T + (bx + bh).
 * Replaces torch.addmm(bx + bh, x.view(T*B,-1), Wx.T) at fastlstm/lstm.py:66-68. */
int fastlstm_gemm_ifgo(const void *x, const void *Wx, const void *bx, const void *bh, void *ifgo,
                       int T, int B, int I, int H, int dtype, void *stream);

/* K2/K3 -- the time loop.  In: ifgo[T,B,4H] holds x.Wx^T+b, out[0]=h_0, cell[0]=c_0.
 * Out: ifgo overwritten with the full pre-activations, out[1..T]=h_t, cell[1..T]=c_t.
 * out, cell: [T+1,B,H]; Wh: [4H,H]; ws: see fastlstm_recurrent_workspace_bytes (forward plan).
 * Replaces the persistent_fwd_kernel launch at fastlstm/lstm.py:131-142
 * (kernel: fastlstm/kernels.py:414-663; H <= 64 takes the single-tile,
 * barrier-free form of fastlstm/kernels.py:672-819). */
int fastlstm_fwd_persistent(void *ifgo, void *out, void *cell, const void *Wh, void *ws,
                            size_t ws_bytes, int T, int B, int H, int dtype, void *stream);

/* K1 + K2/K3 for one layer in one call: the same results as fastlstm_gemm_ifgo followed by
 * fastlstm_fwd_persistent (same arguments, same workspace contract).  Where the XCD-local
 * recurrence leaves CUs without a role (few batch tiles) and those CUs keep up with the recurrence, the
 * workgroups on them compute the input projection inside the same launch, earliest timesteps first, and
 * the recurrence follows them chunk by chunk; otherwise the two stages are launched back to back.  Replaces
 * fastlstm/lstm.py:66-68 together with 131-142. */
int fastlstm_fwd_layer(const void *x, const void *Wx, const void *bx, const void *bh, const void *Wh,
                       void *ifgo, void *out, void *cell, void *ws, size_t ws_bytes, int T, int B, int I,
                       int H, int dtype, void *stream);

/* fastlstm_fwd_layer without a workspace argument and without any allocation.  No counterpart in the
 * reference; it is for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  The recurrence workspace is a static device array of
 * fastlstm_noalloc_scratch_bytes() = 16 MiB inside the library (every GPU the library runs on holds its
 * own copy until the process ends); the call clears the part it needs zeroed itself and calls no
 * hipMalloc/hipFree.  Same results as fastlstm_fwd_layer with a zeroed workspace of
 * min(16 MiB, fastlstm_recurrent_workspace_bytes(forward plan)) bytes -- the kernel choice follows the
 * workspace size as it does there (XCD-local kernels while a slot per timestep fits, else the general
 * ones).  FASTLSTM_ERR_WORKSPACE if the smallest workspace of the shape (plan.ws_bytes) exceeds the array.
 * All calls on one GPU share the array: calls that overlap in time on one GPU (two streams, two threads)
 * race; serialise them.  The XCD-local kernels are only chosen on a device that fastlstm_plan_device has
 * seen (that call probes and may allocate; this one never does).  Set-up: call
 * fastlstm_noalloc_scratch_bytes() once per device, with that device current and outside stream capture,
 * before the first fastlstm_fwd_layer_noalloc there: it looks up the array's device address and creates
 * the pinned status word and the event of the failure reporting and stream ordering described above
 * (without it the entry point still works, looks the address up at its first call -- not a capturable
 * operation -- and reports no failures until some other call has created the status word). */
int fastlstm_fwd_layer_noalloc(const void *x, const void *Wx, const void *bx, const void *bh, const void *Wh,
                               void *ifgo, void *out, void *cell, int T, int B, int I, int H, int dtype,
                               void *stream);
size_t fastlstm_noalloc_scratch_bytes(void);

/* fastlstm_fwd_layer for a forward pass that no reverse pass follows (the reference decides this per
 * call from torch.is_grad_enabled / requires_grad and still stores everything, fastlstm/lstm.py:
 * 507-522): out[1..T] and cell[T] are the same bits as fastlstm_fwd_layer writes; the recurrence
 * does NOT write the gate pre-activations back (ifgo keeps the input projection x.Wx^T + bx + bh)
 * and does not store cell[1..T-1], which stay as the caller left them.  Same arguments, workspace
 * and launch shape; 5 of the 13 bytes per element and timestep the training pass moves are not
 * written.  fastlstm_fwd_stack2_infer is the same for fastlstm_fwd_stack2. */
int fastlstm_fwd_layer_infer(const void *x, const void *Wx, const void *bx, const void *bh, const void *Wh,
                             void *ifgo, void *out, void *cell, void *ws, size_t ws_bytes, int T, int B,
                             int I, int H, int dtype, void *stream);
int fastlstm_fwd_stack2_infer(const void *x, const void *Wx0, const void *bx0, const void *bh0,
                              const void *Wh0, void *ifgo0, void *out0, void *cell0, const void *Wx1,
                              const void *bx1, const void *bh1, const void *Wh1, void *ifgo1, void *out1,
                              void *cell1, void *ws, size_t ws_bytes, int T, int B, int I, int H, int dtype,
                              void *stream);

/* Two stacked layers in one call: the second layer's input is out0[1:] (its input size is H).  The
 * same results as fastlstm_fwd_layer for the first layer followed by fastlstm_fwd_layer for the
 * second.  Where the XCD-local recurrences of BOTH layers fit the device next to each other and
 * leave CUs without a role (fastlstm_fwd_stack2_fused returns 1: e.g. H = 1024, B <= 32), the two
 * layers run in ONE launch: the idle workgroups compute both input projections, the second one
 * chunk by chunk behind the first layer's recurrence, and the second layer's recurrence follows a
 * chunk of timesteps behind the first -- the wall time of one layer instead of two.  Otherwise the
 * layers run one after the other.  ws: fastlstm_stack2_workspace_bytes (ring slots for both layers),
 * zeroed like any recurrent workspace.  Replaces two iterations of the layer loop at
 * fastlstm/lstm.py:685-696 (which the reference runs strictly one after the other, README.md:94). */
int fastlstm_fwd_stack2(const void *x, const void *Wx0, const void *bx0, const void *bh0, const void *Wh0,
                        void *ifgo0, void *out0, void *cell0, const void *Wx1, const void *bx1,
                        const void *bh1, const void *Wh1, void *ifgo1, void *out1, void *cell1, void *ws,
                        size_t ws_bytes, int T, int B, int I, int H, int dtype, void *stream);
size_t fastlstm_stack2_workspace_bytes(const fastlstm_plan *plan, int T, int H, int dtype);
/* 1 if fastlstm_fwd_stack2 runs both layers in one launch for this shape and workspace size on the
 * current device, 0 if it runs them one after the other; negative: fastlstm_status. */
int fastlstm_fwd_stack2_fused(int T, int B, int I, int H, int dtype, size_t ws_bytes);

/* K4 -- the reverse time loop.  In: dout[T,B,H]; dh,dc [B,H] hold the gradients
 * flowing into h_T, c_T; ifgo, cell as written by the forward.  Out: d_ifgo[T,B,4H];
 * dh, dc overwritten with the gradients of h_0, c_0.  ws: see
 * fastlstm_recurrent_workspace_bytes (backward plan).
 * Replaces the lstm_persistent_seq_bwd launch at fastlstm/lstm.py:277-290
 * (kernel: fastlstm/kernels.py:1201-1409). */
int fastlstm_bwd_persistent(const void *dout, void *dh, void *dc, const void *ifgo,
                            const void *cell, void *d_ifgo, const void *Wh, void *ws,
                            size_t ws_bytes, int T, int B, int H, int dtype, void *stream);

/* Two independent recurrences of one shape -- the two directions of a bidirectional layer, whose reverse
 * direction is the same time loop over the reversed sequence -- as ONE launch of the XCD-local kernels where
 * both sets of barrier groups fit the device side by side, else one after the other.  Arguments of recurrence a,
 * then b, as fastlstm_fwd_persistent / fastlstm_bwd_persistent take them; keep_activations = 0 is the inference
 * form.  ws: fastlstm_stack2_workspace_bytes (forward) / fastlstm_stack2_bwd_workspace_bytes (the exchange slots
 * of both recurrences), zeroed like any recurrent workspace.  fastlstm_pair_fused: 1 if the call is one launch
 * for this shape and workspace size on the current device, 0 if not; negative: fastlstm_status.  The reference has
 * no bidirectional layers (README.md:92-94): a host that adds them calls the time loop of
 * fastlstm/lstm.py:102-112 / 277-290 once per direction; these two replace that pair of calls. */
int fastlstm_fwd_persistent_pair(void *ifgo_a, void *out_a, void *cell_a, const void *Wh_a, void *ifgo_b,
                                 void *out_b, void *cell_b, const void *Wh_b, void *ws, size_t ws_bytes, int T,
                                 int B, int H, int dtype, int keep_activations, void *stream);
int fastlstm_bwd_persistent_pair(const void *dout_a, void *dh_a, void *dc_a, const void *ifgo_a,
                                 const void *cell_a, void *d_ifgo_a, const void *Wh_a, const void *dout_b,
                                 void *dh_b, void *dc_b, const void *ifgo_b, const void *cell_b, void *d_ifgo_b,
                                 const void *Wh_b, void *ws, size_t ws_bytes, int T, int B, int H, int dtype,
                                 void *stream);
int fastlstm_pair_fused(int T, int B, int H, int dtype, int backward, size_t ws_bytes);

/* The same for n = 1 ... 4 independent recurrences of one shape, their operands as arrays of n pointers (entry r of
 * each array belongs to recurrence r): the chunks of a wavefront over stacked layers -- launch k runs layer l's
 * chunk k - l of timesteps for every layer l, a time loop started at out[t0] / cell[t0] continuing the sequence --
 * which spreads the layer loop of fastlstm/lstm.py:685-696 (README.md:94: "doesn't exploit num_layer
 * parallelisation") over the device.  One launch where n x the groups of one recurrence fit the XCDs -- XCD-local and
 * register-resident kernels with 16- or 32-row groups, and always for H <= 64, whose
 * workgroups exchange nothing -- (fastlstm_multi_fused), else one recurrence after the other.  ws: fastlstm_multi_workspace_bytes (the exchange
 * slots of n recurrences), zeroed like any recurrent workspace. */
int fastlstm_fwd_persistent_multi(int n, void *const *ifgo, void *const *out, void *const *cell,
                                  const void *const *Wh, void *ws, size_t ws_bytes, int T, int B, int H,
                                  int dtype, int keep_activations, void *stream);
int fastlstm_bwd_persistent_multi(int n, const void *const *dout, void *const *dh, void *const *dc,
                                  const void *const *ifgo, const void *const *cell, void *const *d_ifgo,
                                  const void *const *Wh, void *ws, size_t ws_bytes, int T, int B, int H,
                                  int dtype, void *stream);
int fastlstm_multi_fused(int n, int T, int B, int H, int dtype, int backward, size_t ws_bytes);
size_t fastlstm_multi_workspace_bytes(const fastlstm_plan *plan, int n, int T, int H, int dtype, int backward);

/* K4 + K5 + K6..K9 for one layer in one call: the same results as fastlstm_bwd_persistent,
 * fastlstm_gemm_dx and fastlstm_gemm_wgrad one after the other (same arguments and workspace
 * contracts; dWx and dWh to the rounding of a different summation order).  Where the XCD-local
 * reverse recurrence leaves CUs without a role, the workgroups on those CUs compute dx and the
 * weight gradients (or dx alone, whichever an estimate of their throughput makes the shorter call) inside
 * the same launch, chunk of timesteps by chunk behind the recurrence; otherwise the stages are launched
 * back to back.  dx may be NULL: no gradient of the layer's input is wanted (autograd's needs_input_grad:
 * the first layer of most models) and K5 is skipped, inside the launch and outside it; dWx, dWh and db may
 * be NULL, all three together: the weights are frozen and K6..K9 are skipped.  (The reference computes all
 * of them whatever autograd asks for, fastlstm/lstm.py:524-538.)  Replaces fastlstm/lstm.py:277-290, 294 and
 * 494-501 together. */
int fastlstm_bwd_layer(const void *dout, void *dh, void *dc, const void *ifgo, const void *cell,
                       void *d_ifgo, const void *Wh, const void *Wx, const void *x, const void *h,
                       void *dx, void *dWx, void *dWh, void *db, void *ws, size_t ws_bytes,
                       void *wgrad_ws, size_t wgrad_ws_bytes, int T, int B, int I, int H, int dtype,
                       void *stream);

/* K5 -- dx[T*B,I] = d_ifgo[T*B,4H] . Wx[4H,I].   Replaces fastlstm/lstm.py:294.  (A narrow 16-bit layer, see
 * fastlstm_gemm_dx_wgrad: the streaming pass of that call with dx alone.) */
int fastlstm_gemm_dx(const void *d_ifgo, const void *Wx, void *dx, int T, int B, int I, int H,
                     int dtype, void *stream);

/* The same product with device scratch memory (any size; fp32 partial sums): a dx with too few output tiles
 * to fill the device (T*B*I small against 4H) is split along K where `scratch` holds the partials, else
 * computed as fastlstm_gemm_dx does.  fastlstm_bwd_layer splits the same way into its weight-gradient
 * workspace.  Replaces fastlstm/lstm.py:294. */
int fastlstm_gemm_dx_split(const void *d_ifgo, const void *Wx, void *dx, int T, int B, int I, int H,
                           int dtype, void *scratch, size_t scratch_bytes, void *stream);

/* K6-K9 -- dWx[4H,I] = d_ifgo^T . x,  dWh[4H,H] = d_ifgo^T . h[0..T-1],
 * db[4H] = column sums of d_ifgo; no transposed copy of d_ifgo is made.
 * h: [T+1,B,H] (only slots 0..T-1 are read).  ws: fastlstm_wgrad_workspace_bytes.
 * Replaces Wgrad at fastlstm/lstm.py:494-501. */
int fastlstm_gemm_wgrad(const void *d_ifgo, const void *x, const void *h, void *dWx, void *dWh,
                        void *db, void *ws, size_t ws_bytes, int T, int B, int I, int H,
                        int dtype, void *stream);
size_t fastlstm_wgrad_workspace_bytes(int T, int B, int I, int H, int dtype);

/* K5 and K6-K9 in one call: dx, dWx, dWh, db as fastlstm_gemm_dx_split and fastlstm_gemm_wgrad compute them
 * (dW to the rounding of a different summation order).  For a narrow layer (fp16 / bf16, H <= 64 and
 * I <= 64 in multiples of 16, T*B >= 256) the four results come from ONE pass over d_ifgo -- every
 * product of such a layer is bound by the traffic of d_ifgo, which separate launches read four times;
 * other shapes run the two stages one after the other.  fastlstm_bwd_layer does the same behind a
 * recurrence that leaves no CUs idle for these products.  dx may be NULL, and so may dWx, dWh and db (all
 * three together).  ws: fastlstm_wgrad_workspace_bytes.  Replaces fastlstm/lstm.py:294 and 494-501. */
int fastlstm_gemm_dx_wgrad(const void *d_ifgo, const void *Wx, const void *x, const void *h, void *dx,
                           void *dWx, void *dWh, void *db, void *ws, size_t ws_bytes, int T, int B,
                           int I, int H, int dtype, void *stream);

/* The reverse pass of two stacked layers in one call (suffix 1: upper layer, 0: lower layer; the
 * upper layer's input is out0[1:]).  The same results as fastlstm_bwd_layer for the upper layer
 * followed by fastlstm_bwd_layer for the lower layer with dout = dx1 (dW to the rounding of a
 * different summation order).  dx1 [T,B,H] is the gradient that flows from the upper into the lower
 * layer (written, then read).  Where both XCD-local reverse recurrences fit the device side by side
 * and leave CUs without a role (fastlstm_bwd_stack2_fused returns 1), ONE launch runs both: the idle
 * workgroups compute dx1 chunk by chunk behind the upper recurrence, the lower recurrence follows
 * dx1 a few chunks behind, and the same workgroups accumulate dWx1, dWh1 and compute dx0; the bias
 * gradients follow as separate launches, and so do the lower layer's weight gradients unless wgrad_ws is
 * large enough to park their tiles between chunks.  With few idle workgroups (48 to 64 at H = 768 ... 1024
 * and B = 48 ... 64) they compute dx1 and dx0 only and all four weight gradients follow as launches.  ws: fastlstm_stack2_bwd_workspace_bytes, zeroed like
 * any recurrent workspace; wgrad_ws: at least the larger of the two layers'
 * fastlstm_wgrad_workspace_bytes; with fastlstm_stack2_bwd_wgrad_workspace_bytes (64 MiB at H = I = 1024)
 * the launch takes the lower layer's dWx0, dWh0 too.  dx0 may be NULL (no gradient of the stack's input is
 * wanted: its product is skipped).  Replaces two backward nodes of the layer loop at
 * fastlstm/lstm.py:685-696 (each lstm.py:236-334 + 494-501). */
int fastlstm_bwd_stack2(const void *dout, void *dh1, void *dc1, const void *ifgo1, const void *cell1,
                        void *d_ifgo1, const void *Wh1, const void *Wx1, const void *out1, void *dWx1,
                        void *dWh1, void *db1, void *dx1, void *dh0, void *dc0, const void *ifgo0,
                        const void *cell0, void *d_ifgo0, const void *Wh0, const void *Wx0, const void *x,
                        const void *out0, void *dx0, void *dWx0, void *dWh0, void *db0, void *ws,
                        size_t ws_bytes, void *wgrad_ws, size_t wgrad_ws_bytes, int T, int B, int I, int H,
                        int dtype, void *stream);
size_t fastlstm_stack2_bwd_workspace_bytes(const fastlstm_plan *plan, int T, int H, int dtype);
size_t fastlstm_stack2_bwd_wgrad_workspace_bytes(int T, int B, int I, int H, int dtype);
int fastlstm_bwd_stack2_fused(int T, int B, int I, int H, int dtype, size_t ws_bytes);

/* Which kernel fastlstm_fwd_persistent (backward = 0) / fastlstm_bwd_persistent (1) will launch on
 * the current device for this shape and a workspace of ws_bytes: 0 = the general kernel
 * (exchange through device memory), 1 = the XCD-local kernel (barrier group on one XCD,
 * exchange through its L2; needs the ring workspace of fastlstm_recurrent_workspace_bytes and a
 * device that fastlstm_plan_device has probed; a batch with more tiles than one launch holds runs as
 * several launches over ranges of rows), 2 = the register-resident kernel for H = 1280, 1536, 1792,
 * 2048 with 16-bit elements (barrier groups of H / 16 workgroups over several XCDs, 64 batch rows
 * each; same needs as 1), 3 = the streamed-weights kernel of a hidden size whose W_h does not fit on chip (more
 * than 32 MiB: the reference's RELOAD_WEIGHTS case, fastlstm/lstm.py:70-72).  Negative: fastlstm_status.
 * Diagnostics; no counterpart in the reference. */
int fastlstm_recurrent_kernel_kind(int T, int B, int H, int dtype, int backward, size_t ws_bytes);

/* Rows of the batch that one launch of fastlstm_fwd_persistent / fastlstm_bwd_persistent takes when the
 * batch has more tiles than a launch of kind 1 or 2 holds (the call then runs one launch per range of that
 * many rows, one after the other); 0 when the whole batch is one launch.  A caller whose sequences differ in
 * length (sorted by length, as in a PackedSequence) can cut its batch at these ranges and end each at its own
 * longest sequence.  Negative: fastlstm_status.  Diagnostics; no counterpart in the reference. */
int fastlstm_recurrent_rows_per_launch(int T, int B, int H, int dtype, int backward, size_t ws_bytes);

/* One launch that gets a forward call ready, instead of three fills/copies by the caller: clears the first
 * `zero_bytes` bytes of the workspace (a multiple of 4; see fastlstm_recurrent_workspace_bytes for how many a
 * call needs zeroed) and writes the initial state into slot 0 of out and cell: h0, c0 ([B,H] each, dense), or
 * zeros when both are NULL.  Replaces `out[0] = h_0; cell[0] = c_0` / the zero initialisation of
 * fastlstm/lstm.py:84-90.  A fill kernel, not a memset: the call can be captured into a graph.
 * The same launch gets a reverse call ready: its workspace, and dh / dc ([B,H] each) in the place of out / cell
 * (zeros when no gradient flows into the final state: the two zeros_like of fastlstm/lstm.py:524-527). */
int fastlstm_prepare_forward(void *ws, size_t zero_bytes, void *out0, void *cell0, const void *h0, const void *c0,
                             int B, int H, int dtype, void *stream);

/* Reads the status word the recurrent kernels leave at the start of their
 * workspace; `ws_head` points to a HOST copy of the first 64 bytes.
 * 0 = ok, FASTLSTM_ERR_TIMEOUT = a barrier wait gave up (the kernel still ran
 * to completion, its results are invalid). */
int fastlstm_ws_status(const void *ws_head);

/* Failure reporting without a host synchronisation.  Every device gets one pinned, device-visible status
 * word: from its first fastlstm_plan_device call, or from its first recurrent entry point outside stream
 * capture.  Every recurrent entry point (fastlstm_fwd_persistent, _fwd_layer[_infer|_noalloc],
 * _fwd_stack2[_infer], _fwd/_bwd_persistent_pair, _fwd/_bwd_persistent_multi, _bwd_persistent, _bwd_layer,
 * _bwd_stack2) enqueues, behind its launches, one tiny kernel that looks at the abort flag of the call's
 * workspace (a barrier wait gave up, or a workgroup of an XCD-placed barrier group found itself on another
 * XCD than the placement rule assumes).  If it is raised the kernel
 *   - sets the device's status word: the NEXT recurrent entry on that device returns FASTLSTM_ERR_TIMEOUT
 *     before launching anything and clears the word, and fastlstm_device_status reads it at any time;
 *   - overwrites results of the failed call with NaN -- forward: out[T] and cell[T]; reverse: dh, dc and
 *     the first row of d_ifgo (fastlstm_bwd_persistent, from which every product made of it inherits),
 *     or dh, dc, db, the first timestep of dx and the first row of dWx, dWh (fastlstm_bwd_layer,
 *     _bwd_stack2) -- so that a loss, a gradient scaler or an isfinite check on the results trips in the
 *     same step, although the failing call itself returned FASTLSTM_OK long before.
 * What stays unreported: the last call of a program, if nobody looks at its results or at
 * fastlstm_device_status after synchronising.
 * fastlstm_device_status reads the word of `device` (-1: current): FASTLSTM_OK or FASTLSTM_ERR_TIMEOUT;
 * clear != 0 resets it.  It reflects the calls whose work has completed on the device by now.  No
 * counterpart in the reference (its spin loops are unbounded, fastlstm/kernels.py:546-548). */
int fastlstm_device_status(int device, int clear);

/* (Diagnostics and test hooks -- kernel-family switch, spin limit, clock traces, the step-latency probe --
 * are declared in fastlstm_hip_diag.h.) */
const char *fastlstm_strerror(int status);
const char *fastlstm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FASTLSTM_HIP_H */
