"""Learning-rate policy of the reference's training scripts, feeding the per-launch ``lr``
scalar of the fused optimizer kernels.

Mirror of ``adjust_learning_rate`` in
runtime/image_classification/main_with_runtime.py:532-563 (and its twin in
runtime/translation/main_with_runtime.py): linear warm-up over the first five epochs when
``lr_warmup`` is set, otherwise ``step`` (x0.1 every 30 epochs), ``polynomial`` (power 2)
or ``exponential_decay`` (0.97 ** (epoch / total_epochs)); the stage's base rate comes from
``StageRuntime.get_adjusted_learning_rate`` (runtime/runtime.py:673-680).  The result is
written into every param group, every iteration."""


def learning_rate(stage_base_lr, epoch, total_epochs, lr_policy, step, epoch_length, lr_warmup=False):
    if lr_warmup and epoch < 5:
        return stage_base_lr * float(1 + step + epoch * epoch_length) / (5. * epoch_length)
    if lr_policy == "step":
        return stage_base_lr * (0.1 ** (epoch // 30))
    if lr_policy == "polynomial":
        power = 2.0
        return stage_base_lr * ((1.0 - (float(epoch) / float(total_epochs))) ** power)
    if lr_policy == "exponential_decay":
        decay_rate = 0.97
        return stage_base_lr * (decay_rate ** (float(epoch) / float(total_epochs)))
    raise NotImplementedError(lr_policy)


def adjust_learning_rate(optimizer, epoch, total_epochs, r, lr_policy, step, epoch_length, base_lr,
                         lr_warmup=False, verbose=False):
    """Same argument order as the reference's function, with ``args.lr`` / ``args.lr_warmup``
    passed explicitly instead of read from the script's globals."""
    stage_base_lr = r.get_adjusted_learning_rate(base_lr=base_lr)
    lr = learning_rate(stage_base_lr, epoch, total_epochs, lr_policy, step, epoch_length, lr_warmup)
    if verbose and step % 100 == 0:
        print("Epoch: %d Step %d \tLearning rate: %f" % (epoch, step, lr))
    for param_group in optimizer.param_groups:
        param_group['lr'] = lr
    return lr


def schedule_for(r, base_lr, epoch, total_epochs, lr_policy, epoch_length, lr_warmup=False):
    """``step -> lr`` closure for ``schedule.stage_train_loop(lr_schedule=...)``."""
    stage_base_lr = r.get_adjusted_learning_rate(base_lr=base_lr)
    return lambda step: learning_rate(stage_base_lr, epoch, total_epochs, lr_policy, step, epoch_length, lr_warmup)
