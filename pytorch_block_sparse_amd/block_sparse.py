"""Block-sparse matrix with packed 32x32 blocks; same public interface as the reference's
``pytorch_block_sparse/block_sparse.py`` (classes at :6, :668, :682).

Storage (unchanged, it is the state_dict format, block_sparse.py:58-65):

* ``data`` ``[nnz*bs0, bs1]``: block ``b`` occupies rows ``b*bs0 .. (b+1)*bs0-1`` and holds its
  block of W transposed (:326-331, :412-413);
* int32 buffers ``cols_a [nnz,2]``, ``row_start_ends_a [X+1]`` (CSR), ``rows_b [nnz,2]``,
  ``col_start_ends_b [Y+1]`` (CSC), ``blocks [2*nnz]`` ((col,row) per data block).

What differs: the matmuls run as gfx950 HIP kernels through ``native`` (no CPU path, errors
raise), the index arrays of a GPU mask are built by a device kernel, ``data`` may be
float32 or bfloat16, and matmul results are contiguous ``[tokens, features]`` tensors.
"""
import numpy
import torch
import torch.nn

from . import native


def _as_2tuple(v, what):
    if len(v) != 2:
        raise Exception(f"{what} should be a tuple of 2 ints")
    return int(v[0]), int(v[1])


class BlockSparseMatrixBase(torch.nn.Module):
    """reference: block_sparse.py:6-665."""

    def __init__(self, shape, block_mask, data, block_shape=(32, 32)):
        super().__init__()
        self.int_type = torch.int32
        self.shape = torch.Size(_as_2tuple(shape, "shape"))
        self.block_shape = _as_2tuple(block_shape, "block_shape")
        self.data = torch.nn.Parameter(data)
        self.rebuild(block_mask, callback=False)

    # ------------------------------------------------------------------ hooks (block_sparse.py:27-31)
    def updated_data(self):
        pass

    def get_differentiable_data(self):
        return self.data

    # ------------------------------------------------------------------ pattern
    @staticmethod
    def blocks_count_(shape, block_shape):
        return torch.Size((shape[0] // block_shape[0], shape[1] // block_shape[1]))

    def blocks_count(self):
        return self.blocks_count_(self.shape, self.block_shape)

    def rebuild(self, block_mask, block_ptr=None, callback=True):
        """(Re)build the five index buffers from a [X, Y] block mask.  reference: block_sparse.py:33-76."""
        data = self.data
        bs0, bs1 = self.block_shape
        if block_mask.device != data.device:
            raise Exception(
                "block_mask and data should have same device, got %s and %s" % (block_mask.device, data.device)
            )
        if data.dim() != 2:
            raise Exception("data should be bidimensional, not of shape %s" % (data.shape,))
        if data.shape[1] != bs1:
            raise Exception("data.shape[1] (%d) should be equal to block_shape[1] (%d)" % (data.shape[1], bs1))
        if data.shape[0] % bs0 != 0:
            raise Exception("data.shape[0] (%d) should be a multiple of block_shape[0] (%d)" % (data.shape[0], bs0))
        if data.dtype not in native.SUPPORTED_DTYPES:
            raise Exception("data should be float32 or bfloat16, not of type %s" % data.dtype)
        if tuple(block_mask.shape) != tuple(self.blocks_count()):
            raise Exception(
                "block_mask shape %s does not match the block grid %s" % (tuple(block_mask.shape), tuple(self.blocks_count()))
            )

        n_blocks = data.shape[0] // bs0
        blocks, cols_a, row_start_ends_a, rows_b, col_start_ends_b = self.build_indices(
            block_mask, block_ptr, n_blocks=n_blocks
        )
        if data.shape[0] != cols_a.shape[0] * bs0:
            raise Exception(
                "data.shape[0] (%d) should be equal to cols.shape[0]*block_shape[0] (%d)"
                % (data.shape[0], cols_a.shape[0] * bs0)
            )
        self.register_buffer("cols_a", cols_a)
        self.register_buffer("row_start_ends_a", row_start_ends_a)
        self.register_buffer("rows_b", rows_b)
        self.register_buffer("col_start_ends_b", col_start_ends_b)
        self.register_buffer("blocks", blocks)
        self._plans = {}
        self.validate_indices()
        self.check_ = False
        if callback:
            self.updated_data()

    def build_indices(self, block_mask, block_ptr=None, n_blocks=None):
        """Index arrays of a mask: (blocks, cols_a, row_start_ends_a, rows_b, col_start_ends_b).

        ``block_ptr[i]`` is the data-block id of the i-th nonzero of the mask in row-major order
        (default ``i``).  reference: block_sparse.py:125-153 and :85-123.  A GPU mask is handled
        by the device kernel; a CPU mask (module construction / checkpoint handling on the host)
        by the tensor code below.  Both are bit-exact with the reference's arrays.
        """
        if block_mask.is_cuda:
            if n_blocks is None:
                n_blocks = int(block_mask.sum().item())
            return native.build_indices(block_mask, block_ptr, n_blocks)
        return self._build_indices_host(block_mask.bool(), block_ptr)

    def _build_indices_host(self, mask, block_ptr):
        X, Y = mask.shape
        rc = mask.nonzero(as_tuple=False)  # row-major
        r, c = rc[:, 0], rc[:, 1]
        nnz = rc.shape[0]
        if block_ptr is None:
            block_ptr = torch.arange(nnz, dtype=torch.long)
        else:
            block_ptr = block_ptr.to(dtype=torch.long)
            if block_ptr.numel() != nnz:
                raise Exception(f"block_ptr has {block_ptr.numel()} entries for {nnz} blocks")
            if nnz and (int(block_ptr.min()) < 0 or int(block_ptr.max()) >= nnz):
                raise Exception("block_ptr holds an entry outside [0, n_blocks)")
        it = self.int_type
        zero = torch.zeros(1, dtype=torch.long)
        cols_a = torch.stack([c, block_ptr], 1).to(it)
        row_start_ends_a = torch.cat([zero, mask.sum(1).cumsum(0)]).to(it)
        order = torch.argsort(c * X + r)  # column-major order of the same nonzeros (keys are unique)
        rows_b = torch.stack([r[order], block_ptr[order]], 1).to(it)
        col_start_ends_b = torch.cat([zero, mask.sum(0).cumsum(0)]).to(it)
        blocks = torch.empty((nnz, 2), dtype=torch.long)
        blocks[block_ptr] = torch.stack([c, r], 1)
        return blocks.reshape(-1).to(it), cols_a, row_start_ends_a, rows_b, col_start_ends_b

    def build_coo_block_index(self):
        """[2, nnz] int32 (block_row, block_col) by data-block id.  reference: block_sparse.py:371-403."""
        b = self.blocks.view(-1, 2)
        return torch.stack([b[:, 1], b[:, 0]], 0)

    def block_norm(self, p=2):
        """Norm of each data block.  reference: block_sparse.py:155-157."""
        d = self.data.reshape(-1, self.block_shape[0] * self.block_shape[1])
        return torch.norm(d.float(), p=p, dim=1)

    def block_mask_build(self, block_positions):
        """Boolean [X, Y] mask of a [2, n] list of positions (default: this matrix's).  reference: :159-165."""
        if block_positions is None:
            block_positions = self.build_coo_block_index().long()
        mask = torch.zeros(tuple(self.blocks_count()), dtype=torch.bool, device=self.data.device)
        mask[block_positions[0], block_positions[1]] = True
        return mask

    def block_replace(self, block_replacements):
        """Move data blocks: rows of ``block_replacements`` are (block_row, block_col, data_block_id).

        reference: block_sparse.py:167-219.
        """
        pos = self.build_coo_block_index().long()
        rep = block_replacements.to(dtype=torch.long, device=pos.device).reshape(-1, 3)
        X, Y = self.blocks_count()
        if self.check_:
            refs = torch.zeros(X * Y, dtype=torch.long, device=pos.device)
            refs[pos[0] * Y + pos[1]] = 1
            refs.index_add_(0, rep[:, 0] * Y + rep[:, 1], torch.ones_like(rep[:, 0]))
            worst = int(refs.argmax())
            if int(refs[worst]) > 1:
                raise Exception(f"Block position ({worst // Y},{worst % Y}) was already used")
        pos[:, rep[:, 2]] = rep[:, :2].t()
        mask = self.block_mask_build(pos)
        block_ptr = torch.argsort(pos[0] * Y + pos[1])
        self.rebuild(mask, block_ptr)

    # ------------------------------------------------------------------ constructors
    @classmethod
    def zeros(cls, shape, n_blocks=None, blocks=None, block_shape=(32, 32), device="cuda", dtype=torch.float32):
        """All-zero matrix with ``n_blocks`` random blocks, or the listed ``blocks`` [(row, col), ...], or full.

        reference: block_sparse.py:221-262 (random positions come from numpy's global RandomState, :250).
        """
        shape = _as_2tuple(shape, "shape")
        for i in range(2):
            if shape[i] % block_shape[i] != 0:
                raise Exception(f"Invalid shape: shape[{i}]={shape[i]} %% block_shape[{i}]={block_shape[i]} is not 0.")
        X, Y = cls.blocks_count_(shape, block_shape)
        if n_blocks is None:
            if blocks is not None:
                for b in blocks:
                    for i in range(2):
                        if b[i] * block_shape[i] >= shape[i]:
                            raise Exception(
                                f"Invalid block definition: block[{i}] = {b[i]} : should be < {shape[i] // block_shape[i]}"
                            )
                n_blocks = len(blocks)
            else:
                n_blocks = X * Y
        else:
            assert blocks is None
        if n_blocks > X * Y:
            raise Exception("Too many blocks : %d > %d * %d = %d" % (n_blocks, X, Y, X * Y))
        if blocks is not None:
            positions = numpy.array([b[0] * Y + b[1] for b in blocks], dtype=numpy.int64)
        else:
            positions = numpy.random.choice(X * Y, size=n_blocks, replace=False)
        flat = torch.zeros(X * Y, dtype=torch.bool)
        flat[torch.from_numpy(numpy.asarray(positions, dtype=numpy.int64))] = True
        block_mask = flat.view(X, Y).to(device)
        data = torch.zeros((n_blocks * block_shape[0], block_shape[1]), dtype=dtype, device=device)
        return cls(shape, block_mask, data, block_shape)

    @classmethod
    def ones(cls, shape, n_blocks=None, blocks=None, block_shape=(32, 32), device="cuda", positive=False,
             dtype=torch.float32):
        """reference: block_sparse.py:264-278."""
        ret = cls.zeros(shape, n_blocks, blocks, block_shape, device, dtype=dtype)
        with torch.no_grad():
            ret.data.fill_(1)
        ret.updated_data()
        return ret

    @classmethod
    def randn(cls, shape, n_blocks=None, blocks=None, block_shape=(32, 32), device="cuda", positive=False,
              dtype=torch.float32):
        """reference: block_sparse.py:280-297."""
        ret = cls.zeros(shape, n_blocks, blocks, block_shape, device, dtype=dtype)
        with torch.no_grad():
            ret.data.normal_()
            if positive:
                ret.data.abs_()
        ret.updated_data()
        return ret

    @classmethod
    def from_dense(cls, dense, block_shape=(32, 32), block_count=None, blocks=None, slow=False, out=None):
        """Build from a dense matrix.  reference: block_sparse.py:299-354.

        With ``blocks``, with ``out`` or with every block kept, each data block is gathered from its
        position (:319-344); with a smaller random ``block_count`` the data is, as in the reference,
        just the first ``block_count*bs0*bs1`` scalars of the dense matrix (:345-350).
        """
        bs0, bs1 = block_shape
        full = (dense.shape[0] * dense.shape[1]) // (bs0 * bs1)
        if out is None:
            if blocks is None:
                if block_count is None:
                    block_count = full
            else:
                block_count = None
            ret = cls.zeros(dense.shape, n_blocks=block_count, blocks=blocks, block_shape=block_shape,
                            device=dense.device, dtype=dense.dtype if dense.dtype in native.SUPPORTED_DTYPES
                            else torch.float32)
        else:
            ret = out
        gather = out is not None or blocks is not None or block_count == full
        with torch.no_grad():
            if gather:
                coo = ret.build_coo_block_index().long()
                if slow:
                    for i in range(coo.shape[1]):
                        r, c = int(coo[0, i]), int(coo[1, i])
                        ret.data[i * bs0 : (i + 1) * bs0] = dense[r * bs0 : (r + 1) * bs0, c * bs1 : (c + 1) * bs1].t()
                else:
                    X, Y = ret.blocks_count()
                    tiles = dense.reshape(X, bs0, Y, bs1).permute(0, 2, 3, 1)  # [X, Y, bs1, bs0] = blocks transposed
                    ret.data.copy_(tiles[coo[0], coo[1]].reshape(-1, bs1))
            else:
                n = ret.data.numel()
                ret.data.copy_(dense.flatten()[:n].reshape(ret.data.shape))
        ret.updated_data()
        return ret

    # ------------------------------------------------------------------ conversions
    def to_sparse(self, data_replace=None):
        """Hybrid sparse COO tensor [X, Y, bs0, bs1].  reference: block_sparse.py:405-421."""
        coo = self.build_coo_block_index().long()
        data = self.data if data_replace is None else data_replace
        bs0, bs1 = self.block_shape
        vals = data.reshape(-1, bs1, bs0).transpose(1, 2)
        X, Y = self.blocks_count()
        return torch.sparse_coo_tensor(coo, vals, (X, Y, bs0, bs1))

    def to_dense(self, data_replace=None):
        """Dense [shape] matrix.  reference: block_sparse.py:423-429; element formula :465-476."""
        coo = self.build_coo_block_index().long()
        data = self.data if data_replace is None else data_replace
        bs0, bs1 = self.block_shape
        X, Y = self.blocks_count()
        grid = torch.zeros((X, Y, bs0, bs1), dtype=data.dtype, device=data.device)
        grid[coo[0], coo[1]] = data.detach().reshape(-1, bs1, bs0).transpose(1, 2)
        return grid.permute(0, 2, 1, 3).reshape(self.shape[0], self.shape[1])

    def check_with_dense(self, dense_version):
        """Raise unless every data block equals its dense block.  reference: block_sparse.py:465-476."""
        coo = self.build_coo_block_index().long()
        bs0, bs1 = self.block_shape
        for i in range(coo.shape[1]):
            r, c = int(coo[0, i]), int(coo[1, i])
            mine = self.data[i * bs0 : (i + 1) * bs0, :].t()
            theirs = dense_version[r * bs0 : (r + 1) * bs0, c * bs1 : (c + 1) * bs1]
            if not (mine == theirs).all():
                raise Exception("non matching data")

    def validate_indices(self):
        """Check the five index buffers against each other and against ``data``; raise on the first mismatch.

        Runs where index buffers enter the object: at the end of ``rebuild`` (where the reference calls
        ``sanity_check`` on both compressed lists, block_sparse.py:67-73) and after ``load_state_dict``.
        It covers ``sanity_check``'s conditions (:431-463) and, beyond them, that the start/end lists start
        at 0 and never decrease and that the data-block ids of each list are a permutation of
        ``0..nnz-1``: the kernels index ``data`` and the entry lists with these values.  Shapes and dtypes
        are checked on the host; the value checks run on the buffers' device and are read back once.
        """
        bs0, bs1 = self.block_shape
        X, Y = self.blocks_count()
        nnz = self.data.shape[0] // bs0
        it = self.int_type
        lists = (
            ("cols_a", self.cols_a, "row_start_ends_a", self.row_start_ends_a, X, Y),
            ("rows_b", self.rows_b, "col_start_ends_b", self.col_start_ends_b, Y, X),
        )
        for name, ids, ends_name, ends, n_lists, _ in lists:
            if ids.dim() != 2 or tuple(ids.shape) != (nnz, 2):
                raise Exception("%s should have shape (%d, 2), not %s" % (name, nnz, tuple(ids.shape)))
            if ids.dtype != it:
                raise Exception("%s should be %s, not of type %s" % (name, it, ids.dtype))
            if ends.dim() != 1 or ends.shape[0] != n_lists + 1:
                raise Exception("%s should have shape (%d,), not %s" % (ends_name, n_lists + 1, tuple(ends.shape)))
            if ends.dtype != it:
                raise Exception("%s should be %s, not of type %s" % (ends_name, it, ends.dtype))
        blocks = self.blocks
        if blocks.dim() != 1 or blocks.shape[0] != 2 * nnz or blocks.dtype != it:
            raise Exception("blocks should be %s of shape (%d,), not %s %s" % (it, 2 * nnz, blocks.dtype, tuple(blocks.shape)))
        problems = []   # (message, 0-d bool tensor: True = broken)
        for name, ids, ends_name, ends, _, limit in lists:
            e = ends.long()
            problems.append(("%s should start at 0 and never decrease" % ends_name, (e[0] != 0) | (e[1:] < e[:-1]).any()))
            problems.append(("%s last element should be equal to the block count (%d)" % (ends_name, nnz), e[-1] != nnz))
            if nnz:
                c, b = ids[:, 0].long(), ids[:, 1].long()
                problems.append(("%s holds a block coordinate outside [0, %d)" % (name, limit), (c.min() < 0) | (c.max() >= limit)))
                b_ok = (b >= 0) & (b < nnz)
                seen = torch.zeros(nnz, dtype=torch.long, device=ids.device)
                seen.index_add_(0, b.clamp(0, nnz - 1), b_ok.long())
                problems.append(
                    ("the data block ids of %s should be a permutation of 0..%d" % (name, nnz - 1), (seen != 1).any())
                )
        if nnz:
            b2 = blocks.view(-1, 2).long()
            problems.append((
                "blocks holds a block position outside the %d x %d grid" % (X, Y),
                (b2.min() < 0) | (b2[:, 0].max() >= Y) | (b2[:, 1].max() >= X),
            ))
            # Within one list the coordinates must increase strictly (sorted, no duplicates): the weight-gradient
            # kernels binary-search a row's entries and size their tables for at most one entry per position.
            # And the two compressed lists and `blocks` must describe the same (row, column) for every data block.
            where = {}
            pos = torch.arange(nnz, device=blocks.device)
            for name, ids, ends_name, ends, n_lists, _ in lists:
                e = ends.long().to(blocks.device).clamp(0, nnz)
                owner = torch.searchsorted(e[1:].contiguous(), pos, right=True)   # the list each entry belongs to
                c, b = ids[:, 0].long().to(blocks.device), ids[:, 1].long().to(blocks.device)
                same = owner[1:] == owner[:-1]
                problems.append(("the coordinates of %s should increase strictly within each of its lists" % name,
                                 (same & (c[1:] <= c[:-1])).any()))
                at = torch.full((nnz, 2), -1, dtype=torch.long, device=blocks.device)
                at[b.clamp(0, nnz - 1)] = torch.stack((owner, c), 1)
                where[name] = at
            rc_a = where["cols_a"]                 # (row, column) of every data block according to the row lists
            rc_b = where["rows_b"].flip(1)         # the column lists hold (column, row)
            problems.append(("cols_a and rows_b should hold the same blocks", (rc_a != rc_b).any()))
            problems.append(("blocks should hold the (column, row) of every data block of cols_a", (b2 != rc_a.flip(1)).any()))
        flags = torch.stack([p[1].to(self.blocks.device) for p in problems]).tolist()
        for (message, _), broken in zip(problems, flags):
            if broken:
                raise Exception(message)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        """Index buffers copied in from a checkpoint are validated before any kernel reads them."""
        names = ("blocks", "cols_a", "row_start_ends_a", "rows_b", "col_start_ends_b")
        before = {n: getattr(self, n).clone() for n in names}
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)
        error_msgs = args[4] if len(args) > 4 else kwargs.get("error_msgs")
        self._plans = {}
        try:
            self.validate_indices()
        except Exception as e:  # reported the way torch reports the other problems of a state dict
            # a caller that catches the error must not be left with index buffers no kernel may read
            for n in names:
                cur = getattr(self, n)
                if cur.shape == before[n].shape:
                    cur.copy_(before[n])
                else:
                    setattr(self, n, before[n])
            if error_msgs is None:
                raise
            error_msgs.append("%sindex buffers are inconsistent: %s" % (prefix, e))

    def sanity_check(self, cols, row_end, shape, block_shape):
        """Consistency of one compressed list.  reference: block_sparse.py:431-463."""
        ends = row_end[1:]
        if cols.dim() != 2:
            raise Exception("cols should be bidimensional, not of shape %s" % (cols.shape,))
        if cols.dtype != self.int_type:
            raise Exception("cols should be %s, not of type %s" % (self.int_type, cols.dtype))
        if ends.dim() != 1:
            raise Exception("row_end should be unidimensional, not of shape %s" % (ends.shape,))
        if ends.shape[0] != shape[0] // block_shape[0]:
            raise Exception(
                "row_end.shape[0] (%d) should be equal to shape[0]/block_shape[0] (%d)"
                % (ends.shape[0], shape[0] // block_shape[0])
            )
        if ends.dtype != self.int_type:
            raise Exception("row_end should be %s, not of type %s" % (self.int_type, ends.dtype))
        if cols.shape[0] and int(cols[:, 0].max()) >= shape[1] // block_shape[1]:
            raise Exception("cols max element cannot be larger than shape[1]/block_shape[1]")
        if ends.shape[0] and int(ends[-1]) != cols.shape[0]:
            raise Exception(
                "row_end last element (%d) should be equal to cols count (%d)" % (int(ends[-1]), cols.shape[0])
            )

    def __repr__(self):
        return "%s(shape=%s, cols=%s, row_start_ends_a=%s, data=%s, block_shape=%s)" % (
            self.__class__.__name__,
            self.shape,
            self.cols_a.shape,
            self.row_start_ends_a.shape,
            self.data.shape,
            self.block_shape,
        )

    def multiply_(self, factor):
        with torch.no_grad():
            self.data.multiply_(factor)
        self.updated_data()

    # ------------------------------------------------------------------ the three matmuls
    def flatten_first_dims(self, dense_a):
        """reference: block_sparse.py:580-589."""
        if dense_a.dim() < 2:
            raise Exception(
                f"Invalid dimensions for dense_a {dense_a.shape} : dense_a should have at least 2 dimensions."
            )
        return dense_a.reshape(-1, dense_a.shape[-1]), dense_a.shape[:-1]

    def unflatten_first_dims(self, result, info):
        """reference: block_sparse.py:591-595."""
        if len(info) > 1:
            result = result.view(*info, result.shape[-1])
        return result

    def tensor_prepare(self, t, message=None, transpose=False):
        """Row-major contiguous operand for the kernels (copies only if needed).

        The reference returns (tensor, memory-order flag) and lets the kernel read either order
        (block_sparse.py:480-494); these kernels read row-major only, so any other stride pattern
        is normalised here, which also covers the stride patterns the reference gets wrong (:493-494).
        """
        return t if t.is_contiguous() else t.contiguous()

    def reverse_matmul_(self, dense_a, transpose=True, bias=None):
        """``a @ self.T`` if transpose else ``a @ self`` for 2-D ``a``.  reference: block_sparse.py:496-578."""
        if dense_a.dim() > 2:
            dense_a = dense_a.reshape(-1, dense_a.shape[-1])
        rows, cols = self.shape
        k, n = (cols, rows) if transpose else (rows, cols)
        if dense_a.shape[1] != k:
            raise Exception("Invalid matrices sizes (%d, %d) x (%d, %d)" % (dense_a.shape[0], dense_a.shape[1], k, n))
        dense_a = self.tensor_prepare(dense_a)
        data = self.data.detach()
        if not data.is_contiguous():
            raise Exception("block data must be contiguous")
        plan = self._matmul_plan(bool(transpose), n, k)
        return native.blocksparse_matmul(dense_a, data, plan, n, k, self.cols_a.shape[0], transpose, bias=bias)

    def _matmul_plan(self, transpose, n, k):
        """Kernel schedule of this pattern for one direction, built on first use and kept until the
        index buffers change (rebuild, load_state_dict, move to another device)."""
        if transpose:
            ptr, indices = self.row_start_ends_a, self.cols_a
        else:
            ptr, indices = self.col_start_ends_b, self.rows_b
        plans = self.__dict__.setdefault("_plans", {})
        key = (transpose, ptr.data_ptr(), indices.data_ptr(), ptr._version, indices._version)
        hit = plans.get(transpose)
        if hit is None or hit[0] != key:
            hit = (key, native.blocksparse_matmul_plan(ptr, indices, n, k))
            plans[transpose] = hit
        return hit[1]

    def reverse_matmul(self, dense_a, transpose, bias=None):
        """Any leading dims.  reference: block_sparse.py:597-604."""
        flat, lead = self.flatten_first_dims(dense_a)
        return self.unflatten_first_dims(self.reverse_matmul_(flat, transpose=transpose, bias=bias), lead)

    def matmul_with_output_sparse_support_(self, dense_a, dense_b, overwrite_data=False):
        """Packed blocks of ``a.T @ b`` on this pattern.  reference: block_sparse.py:606-655."""
        if dense_a.shape[0] != dense_b.shape[0] or self.shape[0] != dense_a.shape[1] or self.shape[1] != dense_b.shape[1]:
            raise Exception(
                "Invalid matrices sizes %s^T x %s for a result of shape %s"
                % (tuple(dense_a.shape), tuple(dense_b.shape), tuple(self.shape))
            )
        out = self.data.detach() if overwrite_data else torch.empty_like(self.data, requires_grad=False)
        native.blocksparse_matmul_back(
            self.tensor_prepare(dense_a), self.tensor_prepare(dense_b), self.row_start_ends_a, self.cols_a, out
        )
        return self.data if overwrite_data else out

    def matmul_with_output_sparse_support(self, dense_a, dense_b, overwrite_data=False):
        """reference: block_sparse.py:657-665."""
        flat_a, lead_a = self.flatten_first_dims(dense_a)
        flat_b, lead_b = self.flatten_first_dims(dense_b)
        assert lead_a == lead_b
        return self.matmul_with_output_sparse_support_(flat_a, flat_b, overwrite_data)


class BlockSparseMatrix(BlockSparseMatrixBase):
    """Native 32x32-block matrix.  reference: block_sparse.py:668-679."""

    def __init__(self, shape, block_mask, data, block_shape=(32, 32)):
        if len(shape) != 2 or shape[0] % 32 != 0 or shape[1] % 32 != 0:
            raise Exception("shape should be a tuple of 2 multiples of 32")
        if len(block_shape) != 2 or block_shape[0] != 32 or block_shape[1] != 32:
            raise Exception("block_shape should be (32, 32) for BlockSparseMatrix; use BlockSparseMatrixEmulator")
        super().__init__(shape, block_mask, data, block_shape)


class BlockSparseMatrixEmulator(BlockSparseMatrixBase):
    """Dense-masked emulation for any block shape, pure torch.  reference: block_sparse.py:682-714."""

    def __init__(self, shape, block_mask, data, block_shape):
        super().__init__(shape, block_mask, data, block_shape)
        self.register_parameter("_dense", None)
        self.updated_data()

    def get_differentiable_data(self):
        return self._dense

    def to_dense(self, data_replace=None):
        if data_replace is None:
            return self._dense
        return data_replace * self._mask

    def _update_data_from_dense(self):
        self.from_dense(self._dense, out=self)

    def updated_data(self):
        with torch.no_grad():
            self._dense = torch.nn.Parameter(super().to_dense())
            self._mask = super().to_dense(data_replace=torch.ones_like(self.data)) == 1

    def reverse_matmul(self, dense_a, transpose=True, bias=None):
        m = self._dense * self._mask
        out = dense_a.matmul(m.t() if transpose else m)
        return out if bias is None else out + bias

    def matmul_with_output_sparse_support(self, dense_a, dense_b, overwrite_data=False):
        a = dense_a.reshape(-1, dense_a.shape[-1])
        b = dense_b.reshape(-1, dense_b.shape[-1])
        return a.t().mm(b) * self._mask
