"""The slice of BMTrain's global ``config`` dict (bmtrain/global_var.py:23) that the
hot path reads.  The distributed runtime that normally fills it is not part of this
package: a single-GPU process starts with an empty communicator set and a ZeRO
group of one, and may add ``load_stream`` (a torch.cuda.Stream) when it runs its
own copy stream next to the compute stream."""

config = {
    "zero_size": 1,   # optim_manager.py:68-70 divides the loss scale by this
}
