"""Counterpart of the reference's `construct_envs` (bps_nav/common/env_utils.py:31-118): builds
the rollout generator of a task from a dataset directory and hands the trainer the tensors it
reads after every step.  The reference wraps host arrays with `torch.from_numpy` and copies
them to the GPU every step (ppo_trainer.py:270-284); here the tensors alias the simulator's
device buffers, so rollout storage can take them with device-to-device copies and the sampled
actions can be passed to `step_start` without leaving the GPU (ppo_trainer.py:228, 249).
"""
from collections import OrderedDict

from . import bps_sim

GENERATORS = {"pointnav": bps_sim.PointNavRolloutGenerator, "flee": bps_sim.FleeRolloutGenerator,
              "exploration": bps_sim.ExplorationRolloutGenerator}


class Sync:
    """What the trainer waits on before it reads a group's observations (env_utils.py:24-30).
    There is no renderer: a step's outputs are complete when step_end returns."""

    def __init__(self, envs, idx):
        self._envs = envs
        self._idx = idx

    def wait(self):
        self._envs.wait_for_frame(self._idx)


def construct_envs(task, episodes_folder, asset_path, batch_size, num_worker_groups=4, double_buffered=True, gpu_id=0,
                   seed=0, **kw):
    """Returns (envs, observations, rewards, masks, infos, syncs) with one entry per group, shaped
    as the reference's: rewards [n,1] f32, masks [n,1] u8, infos {name: [n,1] f32},
    observations["pointgoal_with_gps_compass"] [n,2] f32 (PointNav only) -- all on the GPU.
    `episodes_folder` is `<dataset>/<split>/content`, `num_worker_groups` the number of scenes
    resident at once (env_utils.py:61-74); extra keyword arguments go to the generator."""
    task = task.lower()
    if task not in GENERATORS:
        raise ValueError("task must be pointnav, flee or exploration")
    envs = GENERATORS[task](episodes_folder, asset_path, batch_size, num_worker_groups, -1, gpu_id, (64, 64), False, False,
                            double_buffered, seed, True, **kw)
    observations, rewards, masks, infos, syncs = [], [], [], [], []
    for i in range(2 if double_buffered else 1):
        observation = OrderedDict()
        if task == "pointnav":
            observation["pointgoal_with_gps_compass"] = envs.get_polars(i)
        packed = envs.get_infos(i)
        infos.append({k: packed[k].view(-1, 1) for k in packed.dtype.names})
        observations.append(observation)
        rewards.append(envs.get_rewards(i).view(-1, 1))
        masks.append(envs.get_masks(i).view(-1, 1))
        syncs.append(Sync(envs, i))
    return envs, observations, rewards, masks, infos, syncs
