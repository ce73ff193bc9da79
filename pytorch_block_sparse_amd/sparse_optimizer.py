"""Prune-and-regrow of weight blocks during training.

Interface of the reference's ``pytorch_block_sparse/sparse_optimizer.py`` (:158-304): a
``torch.optim.Optimizer`` whose "parameters" are ``BlockSparseMatrix`` objects and whose ``lr``
is the fraction of blocks moved per ``step()``.  Each step drops the lowest-norm blocks of a
matrix, gives their storage to randomly chosen empty positions (``block_replace``), fills them
with small values and clears the attached Adam state of those blocks.
"""
import torch
import torch.optim as optim

from .block_sparse import BlockSparseMatrix


class SparseOptimizerStrategy:
    def run(self, block_sparse_matrix):
        raise NotImplementedError()


class MagnitudeSparseOptimizerStrategy(SparseOptimizerStrategy):
    """reference: sparse_optimizer.py:12-87."""

    def __init__(self, cleanup_ratio, new_coefficients_distribution="uniform", new_coefficients_scale=0.1):
        self.cleanup_ratio = cleanup_ratio
        self.new_coefficients_distribution = new_coefficients_distribution
        self.new_coefficients_scale = new_coefficients_scale

    def initialize_new_blocks(self, old_data, new_data):
        # mean and std stay 0-d tensors on the data's device: nothing here waits for the GPU
        mean, std = old_data.float().mean(), old_data.float().std()
        scale = self.new_coefficients_scale
        if self.new_coefficients_distribution == "gaussian":
            new_data.normal_(mean=0.0, std=1.0)
            new_data.mul_((std * scale).to(new_data.dtype)).add_((mean * scale).to(new_data.dtype))
        elif self.new_coefficients_distribution == "uniform":
            # The reference draws with random_(0, 1), whose only possible value is 0, so its
            # "uniform" blocks are the constant -std*scale (sparse_optimizer.py:31-34).  Kept as is.
            new_data.random_(0, 1)
            new_data -= 0.5
            new_data *= (2 * std * scale).to(new_data.dtype)
        else:
            raise Exception("Unknown new coefficients method %s" % self.new_coefficients_distribution)

    def free_positions(self, bsm, count):
        """`count` distinct empty block positions chosen uniformly at random, as [count, 2] (block row, block column).

        On a GPU the choice is made on the GPU: every position draws a uniform key, occupied positions get a key
        above all others, and the `count` smallest keys win (a uniform random subset in random order, like the first
        `count` entries of a random permutation of the empty positions, reference sparse_optimizer.py:55-56).  The
        number of empty positions follows from the shapes, so nothing is read back.  On the CPU the reference's own
        sequence is kept (torch.randperm over the list of empty positions), so seeded host runs choose as it does.
        """
        mask = bsm.block_mask_build(None)
        X, Y = mask.shape
        n_free = X * Y - bsm.data.shape[0] // bsm.block_shape[0]
        if not mask.is_cuda:
            free = (~mask).nonzero()
            return free[torch.randperm(free.shape[0])[:count]]
        take = min(count, n_free)
        keys = torch.rand(X * Y, device=mask.device)
        keys.masked_fill_(mask.view(-1), 2.0)
        pick = torch.topk(keys, take, largest=False, sorted=True).indices
        return torch.stack([pick // Y, pick % Y], 1)

    def run(self, block_sparse_matrix):
        """reference: sparse_optimizer.py:38-87.  On a GPU every step runs there: block norms, their order, the choice
        of empty positions, the new index buffers (block_replace -> pbs_build_indices) and the new values; the only
        waits are the error checks of rebuild (one status word and one validation flag vector read back)."""
        bsm = block_sparse_matrix
        bs0, bs1 = bsm.block_shape
        order = bsm.block_norm().sort()[1]
        dropped = order[: int(order.shape[0] * self.cleanup_ratio)]

        positions = self.free_positions(bsm, dropped.shape[0])
        bsm.block_replace(torch.cat([positions, dropped.unsqueeze(-1)], -1))

        fresh = torch.zeros(bsm.data.shape[0] // bs0, dtype=torch.bool, device=bsm.data.device)
        fresh[dropped] = True
        fresh = fresh.repeat_interleave(bs0).unsqueeze(-1).expand(-1, bs1).to(bsm.data.dtype)

        new_blocks = torch.zeros_like(bsm.data)
        self.initialize_new_blocks(bsm.data.detach(), new_blocks)
        keep = 1.0 - fresh
        with torch.no_grad():
            bsm.data.mul_(keep).add_(new_blocks * fresh)
        bsm.updated_data()
        return keep


class OptimizerStateUpdater:
    """reference: sparse_optimizer.py:99-124."""

    def __init__(self, optimizer, sparse_object):
        if not isinstance(sparse_object, BlockSparseMatrix):
            raise Exception(f"Unknown sparse_object type {sparse_object}")
        self.optimizer = optimizer
        self.sparse_object = sparse_object

    def update_state_data(self, param, state_keep_mask):
        raise NotImplementedError()

    def update_state(self, state_keep_mask):
        target = self.sparse_object.data
        found = False
        for group in self.optimizer.param_groups:
            for param in group["params"]:
                if param is target:
                    found = True
                    self.update_state_data(param, state_keep_mask)
        return found


class AdamOptimizerStateUpdater(OptimizerStateUpdater):
    """Zero the Adam moments of regrown blocks.  reference: sparse_optimizer.py:127-155."""

    @staticmethod
    def is_compatible(optimizer):
        if isinstance(optimizer, (optim.Adam, optim.AdamW)):
            return True
        try:
            import transformers.optimization as transformers_optim
        except Exception:
            return False
        hf_adamw = getattr(transformers_optim, "AdamW", None)
        return hf_adamw is not None and isinstance(optimizer, hf_adamw)

    def update_state_data(self, param, state_keep_mask):
        state = self.optimizer.state[param]
        for key in state:
            if key in ("exp_avg", "exp_avg_sq", "max_exp_avg_sq"):
                state[key] *= state_keep_mask
            elif key == "step":
                pass  # shared step count; bias correction of the new blocks is slightly off, as in the reference
            else:
                raise Exception(f"Unknown key in Adam parameter state {key}")


class SparseOptimizer(torch.optim.Optimizer):
    """reference: sparse_optimizer.py:158-304."""

    METHODS = ["magnitude"]
    COEFFICIENTS_DISTRIBUTION = ["uniform", "gaussian"]
    allowed_keys = {"lr", "method", "new_coefficients_scale", "new_coefficients_distribution"}

    def __init__(self, sparse_objects, lr=1e-1, method="magnitude", new_coefficients_scale=0.1,
                 new_coefficients_distribution="uniform"):
        if not 0.0 < lr:
            raise ValueError("Invalid learning rate: {}".format(lr))
        defaults = dict(
            lr=lr,
            method=method,
            new_coefficients_scale=new_coefficients_scale,
            new_coefficients_distribution=new_coefficients_distribution,
        )
        super().__init__([{"sparse_objects": sparse_objects}], defaults)
        self.attached_optimizers = []

    @staticmethod
    def sparse_objects(model):
        return [m for _, m in model.named_modules() if isinstance(m, BlockSparseMatrix)]

    def attach_optimizer(self, optimizer):
        if optimizer not in self.attached_optimizers:
            self.attached_optimizers.append(optimizer)

    def add_param_group(self, sparse_objects_group):
        assert isinstance(sparse_objects_group, dict), "param group must be a dict"
        for k in sparse_objects_group:
            if k != "sparse_objects" and k not in self.allowed_keys:
                raise Exception("Unknown cleaning parameter %s" % k)
        objs = sparse_objects_group["sparse_objects"]
        objs = [objs] if isinstance(objs, BlockSparseMatrix) else list(objs)
        sparse_objects_group["sparse_objects"] = objs
        for p in objs:
            if not isinstance(p, BlockSparseMatrix):
                raise Exception("I don't know how to clean this type of object: %s" % p)
        for name, default in self.defaults.items():
            sparse_objects_group.setdefault(name, default)
        if sparse_objects_group["method"] not in self.METHODS:
            raise Exception(f"Invalid Method {sparse_objects_group['method']}")
        if sparse_objects_group["new_coefficients_distribution"] not in self.COEFFICIENTS_DISTRIBUTION:
            raise Exception(
                f"Invalid new coefficients distribution {sparse_objects_group['new_coefficients_distribution']}"
            )
        already = set()
        for group in self.param_groups:
            already.update(group["sparse_objects"])
        if not already.isdisjoint(objs):
            raise ValueError("some parameters appear in more than one parameter group")
        self.param_groups.append(sparse_objects_group)

    def clean(self, p, method, clean_ratio, new_coefficients_scale, new_coefficients_distribution):
        if not isinstance(p, BlockSparseMatrix):
            raise Exception("I don't know how to clean this : %s" % p)
        if method != "magnitude":
            raise Exception(f"Unknowncleaning method {method}")
        strategy = MagnitudeSparseOptimizerStrategy(
            clean_ratio,
            new_coefficients_distribution=new_coefficients_distribution,
            new_coefficients_scale=new_coefficients_scale,
        )
        keep = strategy.run(p)
        if self.attached_optimizers:
            found = False
            for optimizer in self.attached_optimizers:
                if not AdamOptimizerStateUpdater.is_compatible(optimizer):
                    raise Exception(f"unsupported optimizer {optimizer.__class__}")
                found = AdamOptimizerStateUpdater(optimizer, p).update_state(keep) or found
            if not found:
                raise Exception(f"Could not find sparse object {p} in optimizers {self.attached_optimizers}")

    def step(self):
        for group in self.param_groups:
            ratio = group["lr"]
            if ratio == 0.0:
                continue
            for p in group["sparse_objects"]:
                self.clean(
                    p,
                    clean_ratio=ratio,
                    method=group["method"],
                    new_coefficients_scale=group["new_coefficients_scale"],
                    new_coefficients_distribution=group["new_coefficients_distribution"],
                )
