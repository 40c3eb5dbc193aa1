"""TGN mailbox with the interface of the reference's
starrygl/nn/memory/mailbox.py:5-98, its reductions and row moves running in
libsgl_hot.so: `index.unique` + `scatter_max` by timestamp become
sgl_unique_compact + sgl_segment_max_ts, the row selection `mail[idx]` is
sgl_gather, the mailbox write is sgl_scatter_update.

The reference class reads attributes it never sets (`self.num_parts`,
`self.memory_param`, `.accessor`, mailbox.py:41-55); here `mailbox_size` and a
plain tensor are used.  Ties between equal timestamps keep the first event.
"""
import torch

from ...lib import _abi, hot_path
from ...utils.context import DistributedContext


def _ordered_key(ts):
    """int64 keys that sort like the timestamps (float32 or integer)."""
    if ts.dtype.is_floating_point:
        bits = ts.float().contiguous().view(torch.int32).to(torch.int64)
        return torch.where(bits < 0, -(bits & 0x7FFFFFFF) - 1, bits)
    return ts.to(torch.int64)


class mailbox:
    def __init__(self, num_nodes, mailbox_size, dim_out, dim_edge_feat, _next_mail_pos=None,
                 _update_mail_pos=False, device=None):
        self.num_nodes, self.mailbox_size = num_nodes, mailbox_size
        self.dim_out, self.dim_edge_feat = dim_out, dim_edge_feat
        self.device = torch.device(device) if device is not None else DistributedContext.get_default_context().device
        width = 2 * dim_out + dim_edge_feat
        self.mailbox = torch.zeros(num_nodes, mailbox_size, width, device=self.device, dtype=torch.float32)
        self.mailbox_ts = torch.zeros((num_nodes, mailbox_size), dtype=torch.float32, device=self.device)
        self.next_mail_pos = (torch.zeros(num_nodes, dtype=torch.long, device=self.device)
                              if _next_mail_pos is None else _next_mail_pos.to(self.device))
        self.update_mail_pos = _update_mail_pos
        self._hp = hot_path(self.device)
        self._state = self._hp.remap_state(num_nodes)
        self._c_box = self._hp.cache(width * 4, self.mailbox.view(num_nodes * mailbox_size, width))
        self._c_ts = self._hp.cache(4, self.mailbox_ts.view(num_nodes * mailbox_size))

    @property
    def shape(self):
        return (self.num_nodes, self.mailbox_size, 2 * self.dim_out + self.dim_edge_feat)

    def reset(self):
        self.mailbox.fill_(0)
        self.mailbox_ts.fill_(0)
        self.next_mail_pos.fill_(0)

    def move_to_gpu(self):
        return self   # the mailbox lives on the HIP device from the start

    def _latest(self, index, mail, mail_ts):
        """One mail per distinct node: the one with the largest timestamp."""
        hp = self._hp
        index = index.to(self.device, torch.int64).reshape(-1).contiguous()
        (local,), uniq, (u, _) = hp.unique_compact([index], _abi.UNIQUE_SORTED, self._state, True)
        _, arg = hp.segment_max_ts(local, _ordered_key(mail_ts.to(self.device)).contiguous(), u)
        mail = mail.to(self.device, torch.float32).contiguous()
        picked = torch.empty((u, mail.shape[1]), dtype=torch.float32, device=self.device)
        hp.gather(hp.cache(mail.shape[1] * 4, mail), arg, picked)
        return uniq[:u], picked, mail_ts.to(self.device)[arg]

    def set_mailbox_local(self, index, source, source_ts, Reduce_Op=None):
        if Reduce_Op == "max":
            index, source, source_ts = self._latest(index, source, source_ts)
        index = index.to(self.device, torch.int64)
        rows = (index * self.mailbox_size + self.next_mail_pos[index]).contiguous()
        hp = self._hp
        box = self.mailbox.view(self.num_nodes * self.mailbox_size, -1)
        hp.scatter_update(self._c_box, box, None, None, None, rows, source.to(self.device, torch.float32).contiguous())
        hp.scatter_update(self._c_ts, self.mailbox_ts.view(-1), None, None, None, rows,
                          source_ts.to(self.device, torch.float32).contiguous())
        if self.mailbox_size > 1:
            self.next_mail_pos[index] = torch.remainder(self.next_mail_pos[index] + 1, self.mailbox_size)

    def get_update_mail(self, src, dst, ts, edge_feats, mem_src, mem_dst, embedding=None, use_src_emb=False,
                        use_dst_emb=False, block=None, Reduce_score=None):
        dev = self.device
        src, dst = src.to(dev), dst.to(dev)
        index = torch.cat([src, dst]).reshape(-1)
        emb_src = emb_dst = None
        if embedding is not None:
            emb_src, emb_dst = embedding[: src.numel()], embedding[src.numel():]
        a, b = (emb_src if use_src_emb else mem_src), (emb_dst if use_dst_emb else mem_dst)
        src_mail = torch.cat([a, b], dim=1).to(dev)
        dst_mail = torch.cat([emb_dst if use_src_emb else mem_dst, emb_src if use_dst_emb else mem_src], dim=1).to(dev)
        if edge_feats is not None:
            ef = edge_feats.to(dev).to(self.mailbox.dtype)
            src_mail, dst_mail = torch.cat([src_mail, ef], dim=1), torch.cat([dst_mail, ef], dim=1)
        mail = torch.cat([src_mail, dst_mail], dim=0)
        mail_ts = torch.cat((ts, ts), -1).to(dev).to(self.mailbox_ts.dtype)
        return self._latest(index, mail, mail_ts)

    def update_next_mail_pos(self):
        if isinstance(self.update_mail_pos, torch.Tensor):
            nid = torch.where(self.update_mail_pos == 1)[0]
            self.next_mail_pos[nid] = torch.remainder(self.next_mail_pos[nid] + 1, self.mailbox_size)
            self.update_mail_pos.fill_(0)

    def get_message(self, idx):
        return self.mailbox[idx], self.mailbox_ts[idx]
