"""optimus.mapper — the slice of ParallelDpPpEpTpMapper the MoE blocks read.

Reference: optimus/mapper.py:386-456.  The blocks use pmap.ep_ind, pmap.expert_parallelism and
pmap.ep_group (optimus/models/common/moe.py:413-415, :477-483).  Process groups are never
created here: this build runs one GPU's share; with expert_parallelism > 1 the expert window
[ep_ind*NR, (ep_ind+1)*NR) is applied and the exchange of tokens with the other ranks is not
performed.
"""


class ParallelDpPpEpTpMapper:
    def __init__(self, data_parallelism=1, pipeline_parallelism=1, expert_parallelism=1,
                 tensor_parallelism=1, rank=0, create_groups=False, use_pp_first=False):
        if create_groups:
            raise NotImplementedError("process groups are outside the single-GPU hot path")
        self.data_parallelism = self.DP = data_parallelism
        self.pipeline_parallelism = self.PP = pipeline_parallelism
        self.expert_parallelism = self.EP = expert_parallelism
        self.tensor_parallelism = self.TP = tensor_parallelism
        self.rank = rank
        dims = [self.DP, self.PP, self.EP, self.TP]
        order = [0, 1, 2, 3] if not use_pp_first else [1, 0, 2, 3]
        # rank -> (dp, pp, ep, tp): last permuted dimension varies fastest (mapper.py ShapeND)
        idx = [0, 0, 0, 0]
        r = rank
        for d in reversed(order):
            idx[d] = r % dims[d]
            r //= dims[d]
        self.dp_ind, self.pp_ind, self.ep_ind, self.tp_ind = idx
        self.dpep_ind = self.dp_ind * self.EP + self.ep_ind
        self.is_model_parallel = (self.PP > 1) or (self.EP > 1) or (self.TP > 1)
        self.dp_group = -1
        self.tp_group = -1
        self.ep_group = -1
        self.dpep_group = -1
