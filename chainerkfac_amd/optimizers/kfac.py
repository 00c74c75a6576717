"""K-FAC optimizer on the HIP path: the single-GPU ``KFAC`` of the reference
(chainerkfac/optimizers/kfac.py) with the same constructor, hyper-parameters,
phase order and attribute names.  ``DistributedKFAC`` and the communicator's
collectives are not part of this package (one GPU, no inter-GPU traffic).

One step = forward and backward under the function hook (A at forward, G / F at
backward, computed by the SYRK kernels), then for every Fisher block: moving
average -> damping -> inverse -> preconditioning, then the momentum update.
The per-block loop of the reference (``update_kfgrads``) is kept, but damping
and inversion of all blocks are issued as one batch: the blocks are independent,
so the results are those of the sequential loop.
"""
from chainerkfac_amd import device as _dev
from chainerkfac_amd import links
from chainerkfac_amd import ops
from chainerkfac_amd.optimizers import fisher_blocks as FB
from chainerkfac_amd.optimizers.fisher_block import PI_TYPE_TRACENORM


class Hyperparameter(object):
    """Attribute bag shared between the optimizer and its update rules."""

    def __init__(self, parent=None):
        object.__setattr__(self, '_parent', parent)

    def __getattr__(self, name):
        parent = object.__getattribute__(self, '_parent')
        if parent is not None:
            return getattr(parent, name)
        raise AttributeError(name)

    def get_dict(self):
        d = {} if self._parent is None else self._parent.get_dict()
        d.update({k: v for k, v in self.__dict__.items() if k != '_parent'})
        return d


_default_hyperparam = Hyperparameter()
_default_hyperparam.lr = 0.001
_default_hyperparam.lr_pre = 0.001
_default_hyperparam.momentum = 0.9
_default_hyperparam.cov_ema_decay = 0.99
_default_hyperparam.damping = 0.03


def _proxy(name):
    return property(lambda self: getattr(self.hyperparam, name),
                    lambda self, v: setattr(self.hyperparam, name, v))


def fblock_constructor(sub_linkname, sub_link, **kwargs):
    """Fisher block for a link, or None for links K-FAC leaves alone
    (reference kfac.py:19-30)."""
    args = (sub_linkname, sub_link)
    if isinstance(sub_link, links.Linear):
        return FB.FisherBlockLinear(*args, **kwargs)
    elif isinstance(sub_link, links.Convolution2D):
        return FB.FisherBlockConvolution2D(*args, **kwargs)
    elif isinstance(sub_link, links.BatchNormalization):
        if sub_link.gamma is None and sub_link.beta is None:
            return None
        return FB.FisherBlockBatchNormalization(*args, **kwargs)
    return None


def extract(blocks, indices, extractor):
    """Per-rank lists of ``(array, triangular)`` in buffer order: for every rank
    the arrays ``extractor(block)`` yields for the blocks that rank owns, blocks
    in index order (reference kfac.py:456-464).  The result is what
    ``_pack_arrays_to_buffer`` / ``_unpack_arrays_from_buffer`` consume."""
    return [[array for index in local_indices for array in extractor(blocks[index])]
            for local_indices in indices]


class KFACHook(links.FunctionHook):
    """Routes each link-function call to the Fisher block that owns it.  The
    owner is found through the identity of the weight array (a dictionary
    lookup instead of the reference's scan over all blocks, kfac.py:38-48)."""

    def __init__(self, fblocks, lanes=None, pending=None):
        self.fblocks = fblocks
        self.lanes = lanes
        self.pending = pending
        self._owner = {}
        for fb in fblocks:
            fb.pending_covs = pending
            fb.lanes = lanes
            for p in fb.link.params():
                self._owner[id(p.data)] = fb

    def _find(self, func, in_data, out_grad_data=None):
        for a in in_data[1:]:
            fb = self._owner.get(id(a)) if a is not None else None
            if fb is not None and fb.is_mine(func, in_data, out_grad_data):
                return fb
        return None

    # The blocks deal the kernels they launch themselves onto the lanes; a factor that
    # only joins the grouped launch costs its hook call no stream switch.
    def forward_postprocess(self, func, in_data):
        fb = self._find(func, in_data)
        if fb is not None:
            fb.forward_postprocess(func, in_data)

    def backward_preprocess(self, func, in_data, out_grad_data):
        fb = self._find(func, in_data, out_grad_data)
        if fb is not None:
            fb.backward_preprocess(func, in_data, out_grad_data)


class KFACUpdateRule(object):
    """v = momentum * v - lr * kfgrad; param += v (reference kfac.py:51-116)."""

    def __init__(self, parent_hyperparam=None, adjust_momentum=False):
        self.hyperparam = Hyperparameter(parent_hyperparam or _default_hyperparam)
        self.adjust_momentum = adjust_momentum
        self.state = None
        self.t = 0
        self.enabled = True
        self._use_fp32_update = False
        self._fp32_param = None

    def use_fp32_update(self, flag=True):
        """Keep a float32 master copy of a float16 parameter and update that
        (Chainer's UpdateRule.use_fp32_update; reference kfac.py:64-85)."""
        self._use_fp32_update = flag

    def init_state(self, param):
        import torch
        # the momentum kernel works in float32: a float16 parameter always gets a float32
        # velocity and master copy (what the reference does under use_fp32_update)
        self.state = {'v': torch.zeros(param.data.shape, dtype=torch.float32, device=param.data.device)}

    def update(self, param):
        if not self.enabled:
            return
        self.t += 1
        if self.state is None:
            self.init_state(param)
        # gradients of a scaled loss carry the scale (so do the preconditioned
        # ones: G^-1 (s g) A^-1); both are divided back before the update, as
        # Chainer's UpdateRule.update does for ``grad`` and the reference for
        # ``kfgrad`` (kfac.py:72-78)
        import torch
        if param.data.dtype == torch.float16:
            # float32 master copy and float32 gradient (reference kfac.py:64-72, 80-85)
            if self._fp32_param is None:
                self._fp32_param = param.data.float()
            grad = param.kfgrad if getattr(param, 'kfgrad', None) is not None else param.grad
            if grad is None:
                return
            grad = grad.float()
            if param._loss_scale is not None:
                grad = grad / param._loss_scale
            self.update_core(param, self._fp32_param, grad)
            param.data.copy_(self._fp32_param)
            return
        if param._loss_scale is not None:
            # the reference's rule divides ``kfgrad`` in place (kfac.py:76-78), Chainer's base
            # rule, which it then calls, ``grad``: both end up unscaled
            if getattr(param, 'kfgrad', None) is not None:
                param.kfgrad /= param._loss_scale
            if param.grad is not None:
                param.grad /= param._loss_scale
        grad = param.kfgrad if getattr(param, 'kfgrad', None) is not None else param.grad
        if grad is not None and grad.dtype != torch.float32:
            grad = grad.float()      # a float16 gradient of a float32 parameter
        self.update_core(param, grad=grad)

    def batched_job(self, param):
        """What ``update`` would hand to the momentum kernel, for
        ``ops.momentum_update_batched``: the rule's bookkeeping is done here
        (step count, state, float32 master copy), the arithmetic -- division by
        the loss scale, the rule, the float16 copy -- is left to the one launch
        that takes all parameters.  Returns None when there is nothing to update,
        or ``NotImplemented`` when the parameter has to go through ``update``
        (arrays the batched kernel does not take)."""
        import torch
        if not self.enabled:
            return None
        grad = param.kfgrad if getattr(param, 'kfgrad', None) is not None else param.grad
        data = param.data
        if grad is not None and not (
                grad.is_cuda and grad.is_contiguous() and grad.dtype in (torch.float32, torch.float16)
                and data.is_cuda and data.is_contiguous() and data.dtype in (torch.float32, torch.float16)
                and (data.dtype == torch.float16 or grad.dtype == torch.float32)):
            return NotImplemented
        self.t += 1
        if self.state is None:
            self.init_state(param)
        half = data.dtype == torch.float16
        if half and self._fp32_param is None:
            self._fp32_param = data.float()
        if grad is None:
            return None
        lr = self.hyperparam.lr
        lr_pre = self.hyperparam.lr_pre
        momentum = self.hyperparam.momentum
        if self.adjust_momentum and lr < lr_pre:
            momentum *= lr / lr_pre
        return {'param': self._fp32_param if half else data, 'v': self.state['v'], 'grad': grad,
                'param_f16': data if half else None,
                # Chainer's base rule divides ``grad`` of a float32 parameter in place as well
                'raw_grad': param.grad if (not half and grad is not param.grad and param.grad is not None
                                           and param.grad.dtype == torch.float32
                                           and param.grad.is_contiguous()) else None,
                # the reference divides the float32 gradient in place (kfac.py:76-78) and a
                # float16 parameter's through a float32 copy (kfac.py:69-75)
                'write_back': not half, 'key': (float(lr), float(momentum), param._loss_scale)}

    def update_core(self, param, data=None, grad=None):
        if grad is None:
            grad = param.kfgrad if getattr(param, 'kfgrad', None) is not None else param.grad
        if grad is None:
            return
        lr = self.hyperparam.lr
        lr_pre = self.hyperparam.lr_pre
        momentum = self.hyperparam.momentum
        if self.adjust_momentum and lr < lr_pre:
            momentum *= lr / lr_pre
        ops.momentum_update(param.data if data is None else data, self.state['v'], grad.contiguous(), lr,
                            momentum)

    update_core_gpu = update_core


class KFAC(object):

    #: invert batch-norm blocks from their rank-n form when that is exact (see
    #: FisherBlockBatchNormalization.lowrank_inverse_args); False forces the
    #: dense Cholesky path for every block
    bn_lowrank_inverse = True

    #: collect the factors of layers that are too small to fill the GPU (most
    #: 1x1 convolutions' G or A, batch-norm and linear blocks) and compute them
    #: with one grouped launch after the backward pass; False computes every
    #: factor inside its hook call.  Read at ``setup``.
    group_small_factors = True

    #: number of side streams the per-layer factor and preconditioning kernels
    #: are dealt onto (layers are independent of each other and most of their
    #: kernels are too small to fill the GPU alone); 0 keeps everything on the
    #: caller's stream.  Read at ``setup``.  Three is the best count for launches
    #: made from the host: a process has four hardware queues, and with more
    #: streams than queues (the caller's stream, the lanes, the library's own side
    #: streams) independent launches wait behind each other (measured on the
    #: ResNet-50 step: 13.4 ms with three lanes, 14.7 with four).  A step replayed
    #: from a captured HIP graph is fastest with four (12.7 against 13.0 ms).
    lanes = 3

    #: apply the momentum rule of all parameters with one launch per set of
    #: hyperparameters (normally one) instead of one launch per parameter
    batch_param_updates = True

    #: moving averages of all factors and the gradient accumulation of all
    #: parameters as one launch each instead of one per array
    batch_elementwise = True

    def __init__(self, lr=_default_hyperparam.lr, momentum=_default_hyperparam.momentum,
                 cov_ema_decay=_default_hyperparam.cov_ema_decay,
                 damping=_default_hyperparam.damping, stab_coeff=16.0,
                 constructor=fblock_constructor, pi_type=PI_TYPE_TRACENORM, use_cholesky=True,
                 loss_scale=None, adjust_momentum=False, acc_iters=1):
        self.hyperparam = Hyperparameter()
        self.hyperparam.lr = lr
        self.hyperparam.lr_pre = lr
        self.hyperparam.momentum = momentum
        self.hyperparam.cov_ema_decay = cov_ema_decay
        self.hyperparam.damping = damping
        self.pi_type = pi_type
        self.constructor = constructor
        self.adjust_momentum = adjust_momentum
        self.stab_coeff = stab_coeff
        self.fblocks = []
        self.kfhook = None
        self._loss_scale = loss_scale
        self.constructor_kwargs = {
            'cov_ema_decay': self.hyperparam.cov_ema_decay,
            'damping': self.hyperparam.damping,
            'use_cholesky': use_cholesky,
            'pi_type': self.pi_type,
            'stab_coeff': self.stab_coeff,
            'loss_scale': self._loss_scale,
        }
        assert acc_iters >= 1, 'Accumulation iterations should be 1 or larger'
        self.acc_iters = acc_iters
        self.acc_count = 0
        self.acc_aware_iterations = 0
        self.only_pic_update_weight = False
        self.target = None
        self.t = 0
        self.observation = {}
        self._hooks = {'pre': [], 'post': []}

    lr = _proxy('lr')
    lr_pre = _proxy('lr_pre')
    momentum = _proxy('momentum')
    cov_ema_decay = _proxy('cov_ema_decay')
    damping = _proxy('damping')

    # ---- set-up ---------------------------------------------------------
    def setup(self, link):
        self.target = link
        self.t = 0
        # the parameters as of now: walking the link tree costs more than a step's launches
        self._params = list(link.params())
        for param in self._params:
            param.update_rule = self.create_update_rule()
        self.fblocks = []
        for sub_linkname, sub_link in sorted(link.namedlinks(), key=lambda kv: kv[0]):
            fblock = self.constructor(sub_linkname, sub_link, **self.constructor_kwargs)
            if fblock is None:
                continue
            self.fblocks.append(fblock)
        self._lanes = _dev.Lanes(self.lanes)
        self._pending = ops.PendingCovs() if self.group_small_factors else None
        self.kfhook = KFACHook(self.fblocks, self._lanes, self._pending)
        return self

    def finish_covs(self):
        """Joins the side streams the hooks queued factor kernels on and runs
        the grouped launch of the factors that were deferred."""
        self._lanes.join()
        if self._pending is not None:
            self._pending.flush()

    def use_fp32_update(self, flag=True):
        """Chainer's Optimizer.use_fp32_update: float32 master copies for float16
        parameters (this implementation always keeps them; the flag is recorded)."""
        self._use_fp32_update = flag
        for param in self._params:
            if param.update_rule is not None:
                param.update_rule.use_fp32_update(flag)

    def create_update_rule(self):
        return KFACUpdateRule(self.hyperparam, adjust_momentum=self.adjust_momentum)

    def add_hook(self, hook, name=None, timing='pre'):
        self._hooks[timing].append(hook)

    def call_hooks(self, timing='pre'):
        for hook in self._hooks[timing]:
            hook(self)

    def reallocate_cleared_grads(self):
        import torch
        for param in self._params:
            if hasattr(param, 'kfgrad') and param.kfgrad is None:
                param.kfgrad = torch.zeros_like(param.data)
            if param.grad is None:
                param.grad = torch.zeros_like(param.data)

    #: read the device-side failure flags of the previous step (NaN fallback of
    #: the batch-norm blocks, non-positive pivots of the inversions) at the start
    #: of every ``update`` and warn; one small device->host copy per step
    numerics_check = True

    def check_numerics(self):
        """Warns about what the previous step's kernels flagged on the device:
        batch-norm blocks whose preconditioned gradient held a NaN (the raw
        gradient was used, reference batch_normalization.py:21-33) and factors
        whose Cholesky factorisation met a non-positive pivot (the reference's
        NumPy path raises there, its GPU path never looks).  Returns the names of
        the affected links.  Must not be called while a HIP graph is captured."""
        import warnings
        import torch
        flags, owners = [], []
        for fb in self.fblocks:
            nan_flag = getattr(fb, 'nan_flag', None)
            if nan_flag is not None:
                flags.append(nan_flag.reshape(-1))
                owners.append((fb, 'nan'))
            info = getattr(fb, 'inv_info', None)
            if info is not None:
                flags.append(info.reshape(-1))
                owners.extend([(fb, 'pivot')] * info.numel())
        if not flags:
            return []
        host = torch.cat(flags).cpu().tolist()
        bad = []
        for v, (fb, what) in zip(host, owners):
            if not v:
                continue
            bad.append(fb.linkname)
            if what == 'nan':
                warnings.warn('Detected NaN in the kfgrads of the batch normalization layer {}; '
                              '``grad`` was substituted for ``kfgrad``'.format(fb.linkname))
            else:
                warnings.warn('The damped factor of {} is not positive definite in float32 '
                              '(non-positive Cholesky pivot); its inverse is not usable'.format(fb.linkname))
        return bad

    # ---- one step -------------------------------------------------------
    def update(self, lossfun=None, *args, **kwargs):
        if self.numerics_check and self.t > 0:
            self.check_numerics()
        if lossfun is not None:
            for fblock in self.fblocks:
                fblock.acc_state = (self.acc_iters, self.acc_count)
            with self.kfhook:
                use_cleargrads = getattr(self, '_use_cleargrads', True)
                loss = lossfun(*args, **kwargs)
                if use_cleargrads:
                    self.target.cleargrads()
                else:
                    self.target.zerograds()
                if self._loss_scale is not None:
                    (loss * self._loss_scale).backward()
                else:
                    loss.backward()
                # Chainer's backward(loss_scale=...) stamps the scale on every
                # parameter that received a gradient; the update rule divides by it
                for param in self._params:
                    param._loss_scale = self._loss_scale
            del loss
        # the factor kernels of this pass ran on the side streams; the small ones are still to run
        self.finish_covs()

        if self.acc_iters > 1:
            if self.accumulate():
                return

        self.reallocate_cleared_grads()
        self.call_hooks('pre')
        self.t += 1
        self.update_kfgrads(self.fblocks)

        if not self.only_pic_update_weight:
            self.update_params()

        self.reallocate_cleared_grads()
        self.call_hooks('post')
        self.acc_aware_iterations += 1
        self.observation['acc_aware_iterations'] = self.acc_aware_iterations

    def update_params(self):
        """``param.update()`` for every parameter (reference kfac.py:250-252).  With
        ``batch_param_updates`` the K-FAC rules that share their hyperparameters
        run as one launch over all their parameters instead of one each."""
        jobs = {}
        for param in self._params:
            rule = param.update_rule
            job = NotImplemented
            if self.batch_param_updates and type(rule) is KFACUpdateRule:
                job = rule.batched_job(param)
            if job is NotImplemented:
                param.update()
            elif job is not None:
                jobs.setdefault(job['key'], []).append(job)
        for (lr, momentum, loss_scale), group in jobs.items():
            ops.momentum_update_batched(
                [j['param'] for j in group], [j['v'] for j in group], [j['grad'] for j in group], lr, momentum,
                loss_scale, [j['write_back'] for j in group], [j['param_f16'] for j in group])
            if loss_scale is not None:
                ops.div_batched([j['raw_grad'] for j in group if j['raw_grad'] is not None], loss_scale)

    # ---- accumulation over acc_iters micro-batches -----------------------
    def accumulate(self):
        if self.acc_count == 0:
            for param in self._params:
                param.acc_grad = None
            for fblock in self.fblocks:
                fblock.acc_covs = None
        self.accumulate_grads()
        self.accumulate_covs()
        self.acc_count += 1
        if self.acc_count == self.acc_iters:
            self.acc_count = 0
            for param in self._params:
                param.grad = param.acc_grad
            for fblock in self.fblocks:
                fblock.covs = fblock.acc_covs
            return False
        elif self.acc_count < self.acc_iters:
            return True
        raise ValueError('acc_count {} should not be larger than acc_iters {}'.format(
            self.acc_count, self.acc_iters))

    def accumulate_grads(self):
        """acc_grad += grad / acc_iters for every parameter (one launch for those
        that start their sum, one for those that continue it)."""
        first, later = [], []
        for param in self._params:
            if param.grad is None:
                continue
            if getattr(param, 'acc_grad', None) is None:
                buf = getattr(param, '_acc_grad_buf', None)
                if buf is None or buf.shape != param.grad.shape:
                    buf = param._acc_grad_buf = param.grad.new_empty(param.grad.shape)
                param.acc_grad = buf
                first.append((param.grad.contiguous(), buf))
            else:
                later.append((param.grad.contiguous(), param.acc_grad))
        for pairs, b in ((first, 0.0), (later, 1.0)):
            if self.batch_elementwise:
                ops.axpby_batched([x for x, _ in pairs], [y for _, y in pairs], 1 / self.acc_iters, b)
            else:
                for x, y in pairs:
                    ops.axpby(x, y, 1 / self.acc_iters, b)

    def accumulate_covs(self):
        """The covariance kernels already added this micro-batch's factors, scaled
        by 1/acc_iters, onto the blocks' running buffers; publish them."""
        for fblock in self.fblocks:
            fblock.check_attr('covs')
            fblock.acc_covs = list(fblock.covs)

    # ---- moving average -> damping -> inverse -> preconditioning ----------
    def update_kfgrads(self, fblocks):
        self.update_cov_emas(fblocks)
        self.update_invs_batched(fblocks)
        self.precondition(fblocks)

    def update_cov_emas(self, fblocks):
        """``fblock.update_cov_emas()`` for every block (reference kfac.py:306-308); the
        moving averages of the blocks that share a decay run as one launch."""
        self.finish_covs()   # factors computed by the hooks
        averaging = {}
        for fblock in fblocks:
            pairs = fblock.cov_ema_pairs() if self.batch_elementwise else None
            if pairs is None:
                fblock.update_cov_emas()
            else:
                averaging.setdefault(fblock.cov_ema_decay, []).extend(pairs)
        for r, pairs in averaging.items():
            ops.axpby_batched([c for c, _ in pairs], [e for _, e in pairs], r, 1 - r)

    #: run the preconditioning products of all connection blocks as one grouped call
    #: (a few launches for the whole network); False calls every block's
    #: ``update_kfgrads`` on its own
    group_precondition = True

    def precondition(self, fblocks):
        """``fblock.update_kfgrads()`` for every block: the connection blocks' GEMMs as one
        grouped call, the other blocks side by side on the lanes."""
        conn = [fb for fb in fblocks if isinstance(fb, FB.FisherBlockConnection)] \
            if self.group_precondition else []
        norm = [fb for fb in fblocks if isinstance(fb, FB.FisherBlockBatchNormalization)] \
            if self.group_precondition else []
        grouped = set(id(fb) for fb in conn + norm)
        for fblock in fblocks:
            if id(fblock) not in grouped:
                self._lanes.run(fblock.update_kfgrads)
        if norm:
            # all batch-norm blocks in two launches, beside the connection blocks' GEMMs
            operands = [fb.kfgrad_operands() for fb in norm]
            self._lanes.run(lambda: ops.precond_bn_batched(*[[o[i] for o in operands] for i in range(6)]))
            for fb in norm:
                fb.finish_kfgrads()
        if conn:
            operands = [fb.kfgrad_operands() for fb in conn]
            shapes = [(o[0].shape[0], o[1].shape[0], o[3] is not None) for o in operands]
            # a plan per set of persistent buffers (inverses, outputs); the gradient arrays may be
            # new ones every step and go through the plan's table of per-call pointers
            bound = tuple(0 if o[i] is None else o[i].data_ptr() for o in operands for i in (0, 1, 4, 5))
            ops.precond_group(shapes, bound).run(*[[o[i] for o in operands] for i in range(6)])
            for fb in conn:
                fb.finish_kfgrads()
        self._lanes.join()

    def update_invs_batched(self, fblocks):
        """``fblock.update_invs()`` for every block, with all damping kernels and
        all inversions issued together."""
        for fb in fblocks:
            fb.check_attr('cov_emas')
        # blocks with a factor kept as its diagonal (a 1-D array) go their own way
        diagonal = [fb for fb in fblocks if fb.has_diagonal_factor()]
        for fb in diagonal:
            fb.update_invs()
        if diagonal:
            fblocks = [fb for fb in fblocks if not fb.has_diagonal_factor()]
        conn = [fb for fb in fblocks if isinstance(fb, FB.FisherBlockConnection)]
        other = [fb for fb in fblocks if not isinstance(fb, FB.FisherBlockConnection)]
        if conn:
            use_pi = {fb._pi_type == PI_TYPE_TRACENORM for fb in conn}
            if len(use_pi) == 1:
                pis = ops.pi_damp_batched([fb.cov_emas[0] for fb in conn],
                                          [fb.cov_emas[1] for fb in conn],
                                          [fb._rW() for fb in conn], use_pi=use_pi.pop(),
                                          pi_out=self._pi_buffer(len(conn), conn[0].cov_emas[0].device))
                for i, fb in enumerate(conn):
                    fb.pi = pis[i:i + 1]
            else:
                for fb in conn:
                    fb.damp()
        # the other blocks' damping in one launch where they can say what it adds
        batched = [fb for fb in other if hasattr(fb, 'damp_args')]
        if len(batched) > 1:
            args = [fb.damp_args() for fb in batched]
            ops.add_diag_batched([a[0] for a in args], [a[1] for a in args], [a[2] for a in args],
                                 [a[3] for a in args])
        else:
            batched = []
        for fb in other:
            if fb not in batched:
                fb.damp()
        # batch-norm blocks whose factor is this step's rank-n matrix U^T U / n:
        # Woodbury inverse (the same dense result, an n x n Cholesky each)
        lowrank = []
        if self.bn_lowrank_inverse:
            by_batch = {}
            for fb in other:
                args = getattr(fb, 'lowrank_inverse_args', lambda: None)()
                if args is not None:
                    by_batch.setdefault(args[0].shape[0], []).append((fb, args))
            for group in by_batch.values():
                fbs = [fb for fb, _ in group]
                bufs = [fb._inv_buffers()[0] for fb in fbs]
                info = self._info_buffer(len(fbs), bufs[0].device, key='_info_lowrank_{}'.format(
                    group[0][1][0].shape[0]))
                # beside the dense inversions below (a lane of its own; joined at the end)
                self._lanes.run(lambda group=group, bufs=bufs, info=info: ops.bn_lowrank_inverse_batched(
                    [a[0] for _, a in group], [a[1] for _, a in group], [a[2] for _, a in group],
                    [a[3] for _, a in group], outs=bufs, info=info))
                for i, fb in enumerate(fbs):
                    fb.invs = [bufs[i]]
                    fb.inv_info = info[i:i + 1]
                lowrank.extend(fbs)
        done = set(id(fb) for fb in lowrank)
        mats, outs, owners = [], [], []
        for fb in fblocks:
            if id(fb) in done:
                continue
            bufs = fb._inv_buffers()
            mats.extend(fb.cov_emas)
            outs.extend(bufs)
            owners.append((fb, len(bufs)))
        if not mats:
            self._lanes.join()
            return
        outs, info = ops.spd_inverse_batched(mats, outs=outs, info=self._info_buffer(len(mats), mats[0].device))
        self.inv_info = info
        pos = 0
        for fb, n in owners:
            fb.invs = outs[pos:pos + n]
            fb.inv_info = info[pos:pos + n]
            pos += n
        self._lanes.join()

    def _pi_buffer(self, n, device):
        import torch
        buf = getattr(self, '_pi_buf', None)
        if buf is None or buf.numel() != n or buf.device != device:
            buf = self._pi_buf = torch.empty(n, dtype=torch.float32, device=device)
        return buf

    def _info_buffer(self, n, device, key='_info_buf'):
        import torch
        buf = getattr(self, key, None)
        if buf is None or buf.numel() != n or buf.device != device:
            buf = torch.empty(n, dtype=torch.int32, device=device)
            setattr(self, key, buf)
        return buf
