"""Accumulator for the loss dicts of a batch, mirroring `classes/losses.py` of the reference
(same method names and behaviour: sum over conversations, `backward(divisor)`, logging by key)."""
from __future__ import annotations

import torch


class LossDict(dict):
    """The nine-key dict of one conversation, as `calculate_divergence` returns it, that also remembers
    the one fp32 [9] tensor its values are views of (`packed`, in key order; entry 0 mirrors
    `train_loss` without its graph).  `Losses` then accumulates a conversation with one addition
    instead of one per key."""
    packed: torch.Tensor | None = None
    keys_packed: tuple = ()


class Losses:
    """Sums loss dicts across the conversations of a batch (classes/losses.py:16-47), runs the
    backward pass on the summed `train_loss` (:70-79) and logs the other keys (:56-68).

    `logger` is anything with `.log(dict, step=int)` (the reference passes a wandb run); None
    disables logging.
    """

    def __init__(self, logger=None, validation: bool = False):
        self._dict: dict[str, torch.Tensor] = {}
        self._packed: torch.Tensor | None = None      # running sum of LossDict.packed, while every dict added so far had one
        self._packed_keys: tuple = ()
        self._train: torch.Tensor | None = None
        self.validation = validation
        self.device = None
        self.logger = logger
        self.num_steps_accumulated = 0

    def _view(self) -> dict[str, torch.Tensor]:
        """The accumulated values by key, for reading: while only packed dicts have been added, a fresh
        dict of views into the running sum."""
        if self._packed is None:
            return self._dict
        d = {}
        if self._train is not None:
            d["train_loss"] = self._train
        d.update(zip(self._packed_keys[1:], self._packed.unbind(0)[1:]))
        return d

    @property
    def loss_dict(self) -> dict[str, torch.Tensor]:
        """The accumulated values by key: a plain dict that the caller may write into, as the
        reference's attribute is (classes/losses.py:22).  Touching it ends the packed accumulation (the
        running sum is spread out into the dict once; later additions go key by key)."""
        self._unpack()
        return self._dict

    @loss_dict.setter
    def loss_dict(self, value: dict[str, torch.Tensor]) -> None:
        self._dict, self._packed, self._train = value, None, None

    def _unpack(self) -> None:
        if self._packed is not None:
            self.loss_dict = self._view()

    def add_losses(self, new_losses: dict[str, torch.Tensor]) -> None:
        """Every key except `train_loss` is cut from the autograd graph; the first dict is adopted,
        later ones are added key by key (out of place).  Raises ValueError on an empty dict.
        The reference clones as well as detaches (classes/losses.py:35-37); a value that carries no
        graph is only aliased here, since nothing in this class writes into a stored value and a copy
        kernel per key and conversation is most of the host-side cost of a small batch.  Dicts that
        come with their values packed in one tensor (`LossDict`) are summed with one addition for
        the logged keys and one for `train_loss`."""
        if not new_losses:
            raise ValueError("No losses to add to the loss dictionary.")
        self.num_steps_accumulated += 1
        packed = getattr(new_losses, "packed", None)
        if packed is not None and (self._packed is not None or not self._dict) and \
                (self._packed is None or self._packed_keys == new_losses.keys_packed):
            train = new_losses.get("train_loss")
            self._packed = packed if self._packed is None else self._packed + packed
            self._packed_keys = new_losses.keys_packed
            if train is not None:
                self._train = train if self._train is None else self._train + train
            return
        self._unpack()
        for key in list(new_losses):
            if key != "train_loss":
                v = new_losses[key]
                new_losses[key] = v.detach().clone() if v.requires_grad else v.detach()
        if not self._dict:
            self._dict = dict(new_losses)
            return
        for key, value in new_losses.items():
            if key in self._dict:
                self._dict[key] = self._dict[key] + value
            else:
                self._dict[key] = value

    def add_batch(self, batch_losses) -> None:
        """The dicts of all conversations of a batch at once (what `distill_loss_batch` returns): the
        same totals and step count as calling `add_losses` on each in turn, from two launches per
        key (a stack and a sum) -- two for all logged keys together when the dicts are packed --
        instead of one addition per key and conversation.  The order of the float additions differs
        from the sequential form, so the last bit of a logged value may."""
        batch_losses = list(batch_losses)
        if not batch_losses:
            raise ValueError("No losses to add to the loss dictionary.")
        if len(batch_losses) == 1:
            self.add_losses(batch_losses[0])
            return
        keys = list(batch_losses[0])
        if any(list(d) != keys for d in batch_losses):
            for d in batch_losses:                           # differing key sets: the sequential form handles them
                self.add_losses(d)
            return
        self.num_steps_accumulated += len(batch_losses) - 1  # add_losses counts the last one
        if all(getattr(d, "packed", None) is not None for d in batch_losses):
            summed = LossDict()
            summed.packed = torch.stack([d.packed for d in batch_losses]).sum(0)
            summed.keys_packed = batch_losses[0].keys_packed
            if "train_loss" in keys:
                summed["train_loss"] = torch.stack([d["train_loss"] for d in batch_losses]).sum(0)
            else:
                summed[keys[0]] = summed.packed[0]
            self.add_losses(summed)
            return
        summed = {}
        for key in keys:
            vals = [d[key] if key == "train_loss" else d[key].detach() for d in batch_losses]
            summed[key] = torch.stack(vals).sum(0)
        self.add_losses(summed)

    def empty(self) -> None:
        self.loss_dict = {}
        self.num_steps_accumulated = 0

    def log(self, step: int, average: bool = True) -> None:
        if self.logger is None:
            return
        prefix = "Val Loss" if self.validation else "Loss"
        for key, value in self._view().items():
            if key == "train_loss":
                continue
            shown = value / self.num_steps_accumulated if average else value
            self.logger.log({f"{prefix}/{key}": shown}, step=step)

    def backward(self, divisor: int = 1) -> None:
        """`train_loss / divisor` backward, then the key is dropped: the sum over the batch's
        conversations divided by the gradient-accumulation count, not a batch mean."""
        if self._packed is not None:
            if self._train is None:
                raise KeyError("train_loss")                  # a second backward: the key is gone, as in the reference
            loss, self._train = self._train / divisor, None
        else:
            loss = self._dict.pop("train_loss") / divisor
        loss.backward()

    def _scaled(self, fn) -> "Losses":
        out = Losses(self.logger, self.validation)
        out.loss_dict = {k: fn(v) for k, v in self._view().items()}
        out.num_steps_accumulated = self.num_steps_accumulated
        return out

    def __truediv__(self, other):
        if isinstance(other, (int, float, torch.Tensor)):
            return self._scaled(lambda v: v / other)
        return NotImplemented

    def __itruediv__(self, other):
        if isinstance(other, (int, float, torch.Tensor)):
            self.loss_dict = {k: v / other for k, v in self._view().items()}
            return self
        return NotImplemented

    def __mul__(self, other):
        if isinstance(other, (int, float, torch.Tensor)):
            return self._scaled(lambda v: v * other)
        return NotImplemented

    def __imul__(self, other):
        if isinstance(other, (int, float, torch.Tensor)):
            self.loss_dict = {k: v * other for k, v in self._view().items()}
            return self
        return NotImplemented

    def __str__(self) -> str:
        head = " Validation Losses:\n" if self.validation else " Training Losses:\n"
        return head + "".join(f"{k}: {v.item():.4f}\n" for k, v in self._view().items())
