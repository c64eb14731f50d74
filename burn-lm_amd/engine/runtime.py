"""What parts need from the machine: device, activation dtype, and the matrix product.

Matrix products ``x[M,K] @ w[N,K]^T``:
* float32 weights: the hand-written float kernels always (plain fused multiply-adds, no
  reduced-precision matrix mode), whatever the activation dtype.  This is the whole float32 path
  and also what keeps a tensor that a checkpoint stores in 32 bits exact in a bfloat16 run.
* bfloat16 weights, up to 64 rows (decode): the hand-written skinny kernel on the matrix cores that
  streams the weight once (where the width fits its registers: see ops.gemv_mfma_group_limit).  From
  17 rows on, the products that come as partial planes (output and down projection) and, from 33 rows
  on, the gated product run on the kernel whose wavefronts each stream their own stages of K through
  shared memory (ops.gemm_rows): with that many rows the activations cost as much traffic as the
  weights, and its loads never stop for a barrier (see rows_plan and gated_linear).
* bfloat16 weights, 65 to 256 rows, K up to 2048 and few columns (the output projection at the 1B
  width): ops.gemm_rows again, a block for every 64 rows (see mid_rows_ring).
* bfloat16 weights, 65 rows and more, narrow output and long K (the down projection of short
  prompts): partial planes from the hand-written matrix-core kernel (see mid_k_groups).
* bfloat16 weights, many rows (prefill): the library product (hipBLASLt through torch), as the
  reference's engine leaves its matrix products to its tensor library
  (crates/burn-lm-llama/src/nn/attention/mha.rs:124-126).  The gate/up product of a gated
  feed-forward runs instead on the hand-written matrix-core kernel that applies the gating in its
  epilogue (ops.gemm_mfma) where that is faster: for short prompts whose tiles all run at once
  and for long prompts of narrow models whose tiles come in whole rounds (see gated_linear).  With
  BURN_LM_AMD_FUSED_GATE_UP=1 it is used for every prompt of 192 rows and more: it never writes the
  [rows, 2 I] intermediate nor reads it back, but its lower rate eats that gain at wider shapes
  (measured over whole prefills: -6 to +4 % at the 1B shape, -6 to +2 % at 3B, 2-7 % slower at
  8B), so beyond the measured cases it is off unless asked for; =0 leaves every product to the library.
"""
from __future__ import annotations

import os

import torch

from ..csrc import ops

SKINNY_MAX_ROWS = 8
MFMA_SKINNY_MAX_ROWS = 64
# The longest K one group of the row-ring product walks before the sum is better cut into partial planes,
# and up to which that product beats the library's at 65 to 256 rows (a block streams its stages of K one
# after another, so its time grows with K while the library's tiles get longer runs): measured at
# widths of 2048, 3072 and 4096.
RING_GROUP_K = 2048
# The shortest K a group keeps when a short K is cut for more blocks.
RING_MIN_GROUP_K = 512
# Numbers of groups that a skinny product's K may be cut into, the longest stretch of K a group gets where a
# finer cut is to be had, and the least share of the compute units that the last round of blocks should keep busy.
GROUP_CHOICES = (1, 2, 3, 4, 6, 8, 12, 16)
GROUP_MAX_K = 4096
GROUP_MIN_FILL = 0.6
# 65 to 256 rows: the longest K at which the row-ring product with a block for every 64 rows still beats the
# library's and the matrix-core kernel's planes (measured: ahead at 1536, 2048 and 2560, behind at 3072 and 4096).
RING_MID_K = 2560
# The longest K at which the fused q/k/v projection on the row ring beats the library's product followed by the
# rotation kernel (ahead at 5120 and below, 20-29 % behind at 8192).
RING_QKV_K = 6144
# The shortest K a group of the matrix-core kernel's partial planes keeps, and the most rows for which a product
# comes as such planes (every group writes a float32 plane of rows x columns that the next norm reads back: measured
# over whole prompts, 2-5 % faster up to 512 tokens and equal beyond).
MFMA_MIN_GROUP_K = 768
MID_PLANES_MAX_ROWS = 512
# Rows for which the fused gate/up product is used when it is switched on (below, the library is
# ahead by far; above, its better rate on long runs of tiles has made up for the extra pass).
FUSED_GATE_UP_ROWS = (192, 4096)


def rows_plan(N, K, compute_units):
    """(groups of K, columns per block) for a product of 17 to 64 rows that may come as partial
    planes (ops.gemm_rows).  A group spans about RING_GROUP_K of K (measured at the 1B, 3B and 8B layer
    shapes: shorter groups write more planes than they gain, longer ones leave compute units
    idle); 32 columns per block where that gives at most one block per compute unit, else 64;
    and a short K is cut further, down to RING_MIN_GROUP_K, while the blocks still all run at once (a
    second, partial round costs more than the shorter walk along K gains: width 2560, 64 rows, two
    groups 6.8 us, four groups 8.8)."""
    groups = 1
    while groups < 8 and K // (groups * 2) >= RING_GROUP_K:
        groups *= 2
    columns = 32 if -(-N // 32) * groups <= compute_units else 64
    while groups < 8 and K // (groups * 2) >= RING_MIN_GROUP_K and -(-N // columns) * groups * 2 <= compute_units:
        groups *= 2
    return groups, columns


class FusedProjectionPlan:
    """Launch geometry of a projection that a part fuses with work of its own (Runtime.qkv_plan).
    kernel: "rows" (ops.gemm_rows_qkv_rope's geometry: `rows` rows staged per block, `columns` columns
    per block, weights as the checkpoint stores them) or "packed" (ops.gemv_qkv_rope's: the packed
    copy of the weights, all rows in registers)."""
    __slots__ = ("kernel", "columns", "rows")

    def __init__(self, kernel, columns=0, rows=0):
        self.kernel, self.columns, self.rows = kernel, columns, rows

    def __repr__(self):
        return f"FusedProjectionPlan({self.kernel!r}, columns={self.columns}, rows={self.rows})"

    def __eq__(self, other):
        return isinstance(other, FusedProjectionPlan) and (self.kernel, self.columns, self.rows) == (other.kernel, other.columns, other.rows)


class LinearWeight:
    """A bound weight matrix [N, K] and, where the skinny product takes it, its copy packed for that
    product.  The copy is made when a product first asks for it (``packed``): an engine that only ever
    runs prompts and large batches never holds a matrix twice.  ``packable`` says whether there is one to
    be had; ``drop_packed()`` gives its memory back (it is made again on demand)."""

    def __init__(self, w, packable=False, gated=False, packed=None):
        self.w, self.gated = w, gated
        self.packable = bool(packable) or packed is not None
        self._packed = packed
        self.shape, self.dtype = w.shape, w.dtype

    @property
    def packed(self):
        if self._packed is None and self.packable:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("a weight's packed copy would have to be made while a graph is being recorded; a step "
                                   "of this shape has to run once outside a recording first")
            self._packed = ops.pack_weight(self.w, gated=self.gated)
        return self._packed

    @property
    def is_packed(self):
        return self._packed is not None

    def drop_packed(self):
        self._packed = None


class Runtime:
    def __init__(self, dtype=torch.bfloat16, device="cuda:0"):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"activation dtype must be bfloat16 or float32, got {dtype}")
        self.dtype = dtype
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("burn-lm_amd runs on the GPU only (device 'cuda:N'); there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible to this process; burn-lm_amd has no CPU path")
        self.ops = ops
        self._k_groups = {}     # (N, K, M) -> groups of K, as chosen once (see k_groups)
        ops.library()  # fail now, loudly, if the kernel library cannot be had
        ops.arrival_counters(self.device)   # allocated here, before any graph capture can be open
        ops.gemm_mfma_init(self.device)     # likewise: a function attribute is set once per device
        ops.static_scratch_init(self.device)   # likewise: the address of the library's own scratch array
        ops.attn_paged_init(self.device)       # likewise: the shared memory of the generic attention's value tiles
        ops.gemm_rows_init(self.device)        # likewise: the rings of stages of the product for 17 to 64 rows
        self.compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        asked = os.environ.get("BURN_LM_AMD_FUSED_GATE_UP")   # "1": wherever it can run, "0": nowhere, unset: where it is ahead
        self.fused_gate_up_rows = FUSED_GATE_UP_ROWS if asked == "1" else (0, -1)
        self.fused_gate_up_measured = asked != "0"
        self.mid_partials = os.environ.get("BURN_LM_AMD_MID_PARTIALS") != "0"   # "0": the library's products instead
        # most rows for which the skinny kernels take the gated product and the partial planes; above,
        # the matrix-core kernels of short prompts do where their tiles fit (settings for measurements:
        # from 33 rows on those are 1-2 % ahead at some shapes and as much behind at others)
        self.skinny_gated_rows = int(os.environ.get("BURN_LM_AMD_SKINNY_GATED_ROWS", MFMA_SKINNY_MAX_ROWS))
        self.skinny_planes_rows = int(os.environ.get("BURN_LM_AMD_SKINNY_PLANES_ROWS", MFMA_SKINNY_MAX_ROWS))
        # "16" or "32": query rows per wavefront of the prefill attention, whatever the step (for measurements)
        self.prefill_queries = int(os.environ.get("BURN_LM_AMD_PREFILL_TILE", "0") or 0)
        # "0": 17 to 64 rows stay on the packed skinny kernels (for measurements)
        self.rows_ring = os.environ.get("BURN_LM_AMD_ROWS_RING") != "0"

    def empty(self, *shape, dtype=None):
        return torch.empty(*shape, dtype=dtype or self.dtype, device=self.device)

    def weight(self, w, gated=False):
        """Prepares a bound matrix for linear(): bfloat16 matrices may get a packed copy that the
        skinny product streams (made at the first product of up to 16 rows, or of up to 64 where no other
        kernel takes them; it doubles the matrix's memory; the plain copy serves everything else).
        gated=True: w is [gate rows; up rows] of a gated feed-forward and will be used through
        gated_linear(); its packed copy pairs each gate row with its up row."""
        w = w.contiguous()
        N, K = w.shape
        # (a K too long for one group of the skinny product still runs in several, as partial planes; the gated
        # product has no planes)
        packable = w.dtype == torch.bfloat16 and K % 8 == 0 and K >= 8 and (
            ops.gemv_mfma_supported(1, N, K) and N % 16 == 0 if gated else True)
        return LinearWeight(w, packable, gated)

    def k_groups(self, N, K, M=1):
        """Into how many groups a skinny product's K is cut: the fewest whose stretch of K is at most
        GROUP_MAX_K (beyond it a wavefront re-reads its activations for every tile) and whose blocks fill
        at least GROUP_MIN_FILL of their last round on the compute units.  Every block streams its stretch
        of the weights at what one unit can bring, so the product takes as long as the unit with the most
        blocks, and a number of blocks just above a multiple of the units leaves most of the chip idle for
        a block's time; few groups of many wavefronts do better than many of few, and every group is a plane
        that the next norm has to add.  Product and norm together, us at 8 rows (blocks x wavefronts in
        brackets): [4096, 14336] in 4 groups (256x7) 25.1, in 8 (512x4) 28.1; [3072, 3072] in 1 (192x6) 9.4,
        in 4 (384x2) 10.2; [2560, 11008] in 3 (240x8) 15.7, in 8 (432x3) 17.6, in 16 (512x2) 19.9; [1536, 6144]
        in 2 (192x6) 9.4, in 8 (384x2) 11.2; [2048, 8192] in 2 (256x8) 11.4, in 3 (192x6) 12.0, in 4 (512x4) 11.3;
        [2048, 2048] in 1 (128x4) 7.1, in 2 (256x2) 6.6; [8192, 8192] in 2 (256x8) 30.7, in 4 (512x4) 29.8."""
        known = self._k_groups.get((N, K, M))
        if known is None:
            known = self._k_groups[(N, K, M)] = self._choose_k_groups(N, K, M)
        return known

    def _choose_k_groups(self, N, K, M):
        best, best_fill = None, -1.0
        for g in GROUP_CHOICES:
            if g > 1 and K // g < RING_MIN_GROUP_K:
                break
            geometry = ops.gemv_mfma_geometry(M, N, K, g)
            if geometry is None or -(-K // g) > GROUP_MAX_K:
                continue
            blocks = geometry[0]
            fill = blocks / (-(-blocks // self.compute_units) * self.compute_units)
            if fill >= GROUP_MIN_FILL:
                return g
            if fill > best_fill:
                best, best_fill = g, fill
        if best is not None:
            return best
        # no grouping within the bounds: the coarsest one the kernel takes
        return next((g for g in (1, 2, 4, 8, 16, 32, 64) if ops.gemv_mfma_geometry(M, N, K, g) is not None), 64)

    def rows_plan(self, N, K):
        """(groups of K, columns per block) for a product of 17 to 64 rows that may come as partial planes."""
        return rows_plan(N, K, self.compute_units)

    def mid_rows_ring(self, M, N, K, planes):
        """65 to 256 rows, K up to 2048, few columns (the output projection of short prompts and of decode
        steps of many sequences at the 1B width): the product of 17 to 64 rows with a block for every 64
        rows, while all its blocks of 32 columns run at once.  Returns the groups of K (two where that
        still gives every block a compute unit and the caller takes partial planes), 0 for another kernel.
        Measured per call at the 1B shape against the library's product: 6.8-7.2 against 9.8 us at 65-128
        rows, 8.0 against 10.8 at 192, 8.9 against 11.1 at 256; at K = 3072 and 4096 (3B, 8B) equal or
        behind, hence the bound on K."""
        if not (self.rows_ring and MFMA_SKINNY_MAX_ROWS < M <= 256 and K <= RING_MID_K):
            return 0
        blocks = self.rows_ring_blocks(M, N)
        if blocks > self.compute_units:
            return 0
        return 2 if planes and K >= 1024 and blocks * 2 <= self.compute_units else 1

    def rows_ring_blocks(self, M, N, columns=32):
        """Blocks of 64 rows and 32 or 64 columns that ops.gemm_rows and ops.gemm_rows_qkv_rope launch."""
        return -(-N // columns) * -(-M // 64)

    def qkv_plan(self, M, N, K):
        """Which fused projection geometry a position encoding should build on for M rows of width K and
        N = all query, key and value columns, or None (project with linear(), then encode).  The encoding
        only has to check that its own kernel exists for the answer; the thresholds live here.
        17 to 64 rows: the row-ring geometry (per call against the packed kernel with two to four row tiles,
        us: width 1536 at 24 / 32 rows 6.4 / 6.7 against 7.4 / 8.0; width 2048 at 17 / 24 / 32 rows 7.0 / 7.0 / 7.4
        against 7.2 / 7.8 / 8.6; width 3072 8.5-9.2 against 16.5-21.8; whole decode steps at batch 17 to 64 of
        the 3B and 8B shapes 2-6 % faster); 33 to 64 rows as two blocks of 32 while both sets run at once (1B
        shape: 7.8-8.2 against 9.3-9.8 us).  65 to 256 rows: a block for every 64
        rows, 32 columns per block while those blocks all run at once, else 64 while there are at most one
        and a half per compute unit (per layer against the library's product and the rotation kernel: 1B
        shape 10 against 14-16 us at 65-128 rows, 13.3 against 21 at 192, 13.6 against 16 at 256; 3B 16-17
        against 18-27 at 65-192, 28.5 against 33 at 256; 8B 21-24.5 against 28-31 at 65-128, 36 against 39
        at 192, 38.5 against 46 at 256).  Up to 16 rows, and whenever the row-ring kernel is not to be
        had: the packed geometry."""
        if self.rows_ring and K <= RING_QKV_K:
            if 16 < M <= MFMA_SKINNY_MAX_ROWS:
                halves = M > 32 and self.rows_ring_blocks(64, N) * 2 <= self.compute_units
                return FusedProjectionPlan("rows", 32, 32 if halves else 64)
            if MFMA_SKINNY_MAX_ROWS < M <= 256:
                if self.rows_ring_blocks(M, N) <= self.compute_units:
                    return FusedProjectionPlan("rows", 32, 64)
                if self.rows_ring_blocks(M, N, 64) * 2 <= self.compute_units * 3:
                    return FusedProjectionPlan("rows", 64, 64)
        if M <= MFMA_SKINNY_MAX_ROWS:
            return FusedProjectionPlan("packed")
        return None

    def mid_planes_plan(self, M, N, K):
        """More than 32 rows, narrow output, long K (the down projection, the output projection of wide models): the
        product as partial planes of the matrix-core kernel over groups of K (the block's next norm sums the
        planes).  -> (groups, tile), or (0, None) for the library's product.  Of the 128x128 and 128x64 tiles
        with eight, four or two groups of at least MFMA_MIN_GROUP_K, the one whose blocks come closest to one
        per compute unit without exceeding that, the larger tile on a tie, and nothing if even that leaves half the
        units idle.  Measured at 128 rows (us, chosen / library): widths 2560, 5120 and 8192 with an inner size of
        11008: 22.4 / 57.6, 37.5 / 60.9, 45.4 / 67.2; width 1536: 14.5 / 21.9; a tie (width 2560, 160 blocks): 128x128
        in eight groups 22.4, 128x64 in four 25.9.  Over whole prompts of 65 to 128 tokens: 6 % faster at the
        Llama-3.2-1B shape, 19 % at 3B, 21 % at 8B (the library's product of few rows and a long K streams the
        weights at a quarter of the memory rate); 2-5 % up to 512 tokens, where two groups still fit; equal beyond."""
        best = (0, None, 0)
        if M > MID_PLANES_MAX_ROWS:
            return 0, None
        for tile, tn in (((128, 128, 4), 128), ((128, 64, 6), 64)):
            tiles = -(-M // 128) * -(-N // tn)
            for g in (8, 4, 2):
                blocks = tiles * g
                if K // g >= MFMA_MIN_GROUP_K and self.compute_units // 2 <= blocks <= self.compute_units and blocks > best[2]:
                    best = (g, tile, blocks)
        return best[0], best[1]

    def mid_k_groups(self, M, N, K):
        """Groups of K of mid_planes_plan (0: the library's product)."""
        return self.mid_planes_plan(M, N, K)[0]

    def linear(self, x, w, out_dtype=None, out=None, partials=False):
        """x [M,K] @ w[N,K]^T -> [M,N] in out_dtype (default: the activation dtype).  w: a
        LinearWeight from weight(), or a plain tensor.  partials=True allows the result to come as
        float32 [groups, M, N] partial products (the caller hands it to a norm's add, which sums
        them); it is used for narrow outputs in decode."""
        packable, holder = False, None
        if isinstance(w, LinearWeight):
            holder, w = w, w.w
            packable = holder.packable and not holder.gated   # a gated copy has its rows re-ordered
        M, K = x.shape
        N = w.shape[0]
        out_dtype = out_dtype or self.dtype
        planes = partials and out is None       # the result may come as float32 partial planes
        if w.dtype == torch.float32 or x.dtype == torch.float32:
            if out is None:
                out = torch.empty(M, N, dtype=out_dtype, device=x.device)
            if M <= SKINNY_MAX_ROWS and x.dtype == w.dtype == out_dtype == torch.float32 and K % 8 == 0 \
                    and x.stride(0) % 8 == 0:
                return ops.gemv_skinny(x, w, out)
            return ops.gemm_tiled(x, w, out)
        aligned = K % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
        if (M > MFMA_SKINNY_MAX_ROWS and aligned and x.dtype == w.dtype == torch.bfloat16 and x.stride(1) == 1
                and w.is_contiguous() and out_dtype == torch.bfloat16):
            groups = self.mid_rows_ring(M, N, K, planes=planes)
            if groups > 1:
                return ops.gemm_rows(x, w, torch.empty(groups, M, N, dtype=torch.float32, device=x.device), columns=32)
            if groups == 1:
                return ops.gemm_rows(x, w, out if out is not None else torch.empty(M, N, dtype=out_dtype, device=x.device),
                                     columns=32)
        plain_bf16 = aligned and x.dtype == w.dtype == torch.bfloat16 and x.stride(1) == 1 and w.is_contiguous()
        if planes and self.mid_partials and M > self.skinny_planes_rows and plain_bf16:
            groups, tile = self.mid_planes_plan(M, N, K)
            if groups:
                return ops.gemm_mfma(x, w, torch.empty(groups, M, N, dtype=torch.float32, device=x.device), tile=tile)
        if (planes and self.rows_ring and 16 < M <= MFMA_SKINNY_MAX_ROWS and plain_bf16
                and (M > 32 or K <= 4096 or -(-N // 32) * 8 <= 3 * self.compute_units)):
            # 17 to 64 rows as partial planes (measured against the packed skinny kernel at the 1B, 3B and 8B
            # shapes: output projection 15-35 % faster at every row count, down projection 25-40 % at K = 8192 of
            # the 1B width, equal to 10 % at the wider ones from 33 rows on).  Up to 32 rows: where K is short or the
            # output narrow (up to 96 blocks of 32 columns on 256 units: widths 1536 and 2560 with inner sizes of
            # 6144 and 11008 at 32 rows 6.2-9.3 us against 8.1-12.0); a wide output with a long K stays with the
            # packed kernel there (equal to 8 % ahead)
            groups, columns = self.rows_plan(N, K)
            if M > 32 and self.mid_partials and -(-N // columns) * groups > self.compute_units:
                # more blocks than compute units even with 64 columns each (a long K under a wide output): the
                # matrix-core kernel's planes where they fill the chip (width 8192, K = 11008, 64 rows: 42.6 against 46.3 us)
                g2, tile = self.mid_planes_plan(M, N, K)
                if g2:
                    return ops.gemm_mfma(x, w, torch.empty(g2, M, N, dtype=torch.float32, device=x.device), tile=tile)
            if groups > 1:
                return ops.gemm_rows(x, w, torch.empty(groups, M, N, dtype=torch.float32, device=x.device), columns=columns)
        if packable and M <= MFMA_SKINNY_MAX_ROWS and aligned:
            if planes:
                groups = self.k_groups(N, K, M)
                if groups > 1:
                    return ops.gemv_mfma(x, holder.packed, torch.empty(groups, M, N, dtype=torch.float32, device=x.device), K)
            if ops.gemv_mfma_supported(M, N, K):
                if out is None:
                    out = torch.empty(M, N, dtype=out_dtype, device=x.device)
                return ops.gemv_mfma(x, holder.packed, out, K)
        if out is None:
            out = torch.empty(M, N, dtype=out_dtype, device=x.device)
        if (out_dtype == torch.float32 and M > 32 and aligned and x.dtype == w.dtype == torch.bfloat16
                and x.stride(1) == 1 and w.is_contiguous() and out.stride(1) == 1 and N * K * 2 < 1 << 32):
            # float32 results (logits) for more rows than one skinny product takes at this width (more than 64,
            # or more than 32 where K is above 2048): the matrix-core kernel with a float output, which reads
            # the weights once.  Measured per call with a vocabulary of 128,256 against the skinny product in
            # chunks of rows (us): width 2048, 65 / 128 / 256 rows: 141 / 156 / 189 against 202 / 230 / 453;
            # width 3072, 33-64 rows: 154-169 against 268-298; width 4096: 233-238 against 329-350, 65-128 rows
            # 240-252 against 509-687; the library's product with a float output: equal to 5 % behind.
            return ops.gemm_mfma(x, w, out, tile=(128, 128, 4) if M <= 128 else (256, 128))
        if packable and aligned and out_dtype == torch.float32:
            # 17 to 32 rows at a K above 4096: the most rows the skinny product does take at a time (16); the
            # weights stream once per chunk, which still beats the plain tiled kernel by far
            chunk = next((c for c in (64, 32, 16) if ops.gemv_mfma_supported(c, N, K)), 0)
            if chunk:
                for r in range(0, M, chunk):
                    ops.gemv_mfma(x[r:r + chunk], holder.packed, out[r:r + chunk], K)
                return out
        if M <= SKINNY_MAX_ROWS and aligned:
            return ops.gemv_skinny(x, w, out)
        if out_dtype == torch.bfloat16:
            return torch.matmul(x, w.t(), out=out)
        # float32 logits from bfloat16 operands with many rows: own kernel (float accumulation)
        return ops.gemm_tiled(x, w, out)

    def _gated_by_library(self, M, K, inner):
        """17 to 64 rows of a gated product that are better left to the library's product and the gating kernel:
        from 33 rows on where K is beyond 4096 (measured at widths 5120 and 8192 with inner sizes of 6144 to 28672:
        6-23 % ahead of the row ring, whose blocks each walk all of K, and of the matrix-core tiles of short
        prompts) or the row ring would take more than two rounds of blocks (width 2560 with an inner size of
        28672: 66.9 against 74.6 us); up to 32 rows where K is beyond what the packed kernel takes and the row
        ring's blocks do not all run at once (width 5120, inner size 11008: 51.6 against 57.7)."""
        if M > 32:
            return K > 4096 or -(-inner // 32) > 2 * self.compute_units
        return K > 4096 and -(-inner // 32) > self.compute_units

    def gated_linear(self, x, w):
        """silu(x gate^T) * (x up^T) for w = [gate rows; up rows] ([2I, K]) -> [M, I].  With few rows
        in bfloat16 the gating is fused into the product (weight(w, gated=True) pairs the rows for
        it); otherwise the product is followed by the gating kernel."""
        M, K = x.shape
        inner = w.shape[0] // 2
        plain = w.w if isinstance(w, LinearWeight) else w
        fusable = (x.dtype == plain.dtype == self.dtype == torch.bfloat16 and K % 8 == 0 and x.stride(1) == 1
                   and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and plain.is_contiguous())
        by_library = 16 < M <= MFMA_SKINNY_MAX_ROWS and self._gated_by_library(M, K, inner)
        if fusable and self.rows_ring and 16 < M <= MFMA_SKINNY_MAX_ROWS and not by_library and (
                M > 32 or -(-inner // 32) <= self.compute_units * (2 if K <= RING_GROUP_K else 1)):
            # 33 to 64 rows (measured against the packed skinny kernel: 4-15 % faster at the 1B and 3B shapes, and
            # at wider ones in place of the library's product, which the packed kernel's registers leave them to);
            # from 17 rows on where the blocks come in one round, or in two where K is short (us at 17 / 24 / 32
            # rows against the packed kernel: width 2048, inner 8192: 14.0 / 14.3 / 14.3 against 16.4 / 17.7 / 18.2;
            # width 1536: 11.8 / 11.9 / 12.0 against 13.3 / 14.1 / 14.6; 3B: 10-15 %)
            return ops.gemm_rows(x, plain, torch.empty(M, inner, dtype=self.dtype, device=x.device), gated=True)
        if (isinstance(w, LinearWeight) and w.packable and w.gated and x.dtype == torch.bfloat16 and not by_library
                and M <= self.skinny_gated_rows and ops.gemv_mfma_supported(M, w.shape[0], K)
                and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0):
            out = torch.empty(M, inner, dtype=self.dtype, device=x.device)
            return ops.gemv_mfma(x, w.packed, out, K, gated=True)
        if fusable and self.fused_gate_up_measured and M > MFMA_SKINNY_MAX_ROWS:
            # Short prompts: when all tiles of the product run at once (one block per compute unit,
            # most of the units busy), the fused kernel with a deep ring of stages streams the
            # weights faster than the library product and the gating pass after it (measured at
            # 65 to 320 rows: 5-25 % at widths of 1536 to 3072, 4 % at 4096; with a second round
            # of tiles the library is ahead).  The narrower tile first: it spreads over more units.
            m128 = -(-M // 128)
            for tile, pairs in (((128, 64, 6), 32), ((128, 128, 4), 64)):
                blocks = m128 * -(-inner // pairs)
                if self.compute_units // 4 <= blocks <= self.compute_units:
                    return ops.gemm_mfma(x, plain, torch.empty(M, inner, dtype=self.dtype, device=x.device),
                                         gated=True, tile=tile)
            # 256x128 tiles that make one round on at least three quarters of the compute units, with rows
            # that fill their tiles to 85 % and more: measured against the library's product and the gating
            # kernel 11-16 % faster with a full round (512 rows of an inner size of 8192 at widths 2048 and
            # 3072; 900 and 1,024 rows of an inner size of 4096), 6 % with three quarters of one (700 and 768
            # rows, inner 4096); rows that fill their tiles less (320, 520, 600) are equal or 5 % behind, and
            # one and a half rounds and more 15-30 % behind.
            m256 = -(-M // 256)
            blocks = m256 * -(-inner // 64)
            if M > 256 and M * 20 >= m256 * 256 * 17 and self.compute_units * 3 // 4 <= blocks <= self.compute_units:
                return ops.gemm_mfma(x, plain, torch.empty(M, inner, dtype=self.dtype, device=x.device),
                                     gated=True, tile=(256, 128))
            # Long prompts: with whole rounds of 256x256 tiles (as many blocks as compute units, or a
            # multiple) and a narrow model the fused kernel is ahead of the library over the whole
            # prefill (width 2048: 2-4 % at 1,024 and 2,048 rows, 0.5-0.8 % at 3,072 and 4,096; behind by
            # 2-6 % with a partial last round, and at width 3072 behind from 1,536 rows on).  Beyond
            # 4,096 rows the library's large tiles are ahead (whole prefill of 8,192 tokens 19.4 ms
            # against 20.7, of 16,384 tokens 47.9 against 49.0).
            if K <= RING_GROUP_K and 256 <= M <= 4096 and (-(-M // 256) * -(-inner // 128)) % self.compute_units == 0:
                return ops.gemm_mfma(x, plain, torch.empty(M, inner, dtype=self.dtype, device=x.device),
                                     gated=True, tile=(256, 256))
        if fusable and self.fused_gate_up_rows[0] <= M <= self.fused_gate_up_rows[1]:
            # the largest tile that still gives every compute unit a block (a tile of n columns holds n / 2 gated pairs)
            m256 = -(-M // 256)
            tile = ((256, 256) if m256 * -(-inner // 128) >= self.compute_units else
                    (256, 128) if m256 * -(-inner // 64) >= self.compute_units else (128, 128))
            return ops.gemm_mfma(x, plain, torch.empty(M, inner, dtype=self.dtype, device=x.device), gated=True, tile=tile)
        gu = self.linear(x, plain)
        act = torch.empty(M, inner, dtype=gu.dtype, device=x.device)
        ops.swiglu(gu, act)
        return act
