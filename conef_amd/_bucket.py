"""Small helpers shared by the hooks: GradBucket accessors that accept both the current
torch spelling (buffer/gradients/index/is_last) and the one the reference was written against
(get_tensor/get_per_parameter_tensors/get_index/is_the_last_bucket_to_allreduce, e.g.
communication/powerSGD_hook.py:343,386,355,244), and a completed Future."""
import torch
import torch.distributed as dist


def _call(bucket, new, old):
    fn = getattr(bucket, new, None)
    if fn is None:
        fn = getattr(bucket, old)
    return fn()


def buffer(bucket):
    return _call(bucket, "buffer", "get_tensor")


def gradients(bucket):
    return _call(bucket, "gradients", "get_per_parameter_tensors")


def index(bucket):
    return _call(bucket, "index", "get_index")


def is_last(bucket):
    return _call(bucket, "is_last", "is_the_last_bucket_to_allreduce")


def group_and_size(process_group):
    """(group, world_size).  Without an initialised process group the world is one rank."""
    if process_group is not None:
        return process_group, process_group.size()
    if dist.is_available() and dist.is_initialized():
        return dist.group.WORLD, dist.group.WORLD.size()
    return None, 1


def completed_future(tensor):
    """A Future already holding ``tensor``; aware of the tensor's device so that DDP orders its
    own stream after the kernels enqueued by the hook."""
    fut = torch.futures.Future(devices=[tensor.device]) if tensor.is_cuda else torch.futures.Future()
    fut.set_result(tensor)
    return fut


def allreduce_fut(group, tensor, world_size):
    """Averaging all-reduce as a Future (what default._allreduce_fut does in the reference).
    At world size 1 the sum is the tensor itself and the division is by one."""
    if world_size == 1:
        return completed_future(tensor)
    tensor.div_(world_size)
    return dist.all_reduce(tensor, group=group, async_op=True).get_future().then(lambda f: f.value()[0])
