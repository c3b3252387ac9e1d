"""Process-wide device context (reference: flash3dxfmr/psh/dev_context.py:9-34)."""
from ..lib import pshattn

DEV_MGR = pshattn.DeviceManagerSingleton.instance()
_STATE = {"trace": False}


def get_dev_manager():
    return DEV_MGR


def init_dev(dev_id: int):
    assert isinstance(dev_id, int), f"Expect dev_id is an int, got {type(dev_id)}"
    DEV_MGR.init_dev_info(dev_id)


def get_sync_stream():
    return DEV_MGR.get_sync_stream()


def set_sync_stream(is_syncing: bool):
    return DEV_MGR.set_sync_stream(is_syncing)


def set_nvtx(flag: bool):
    """Range markers around modules (roctx through torch.cuda.nvtx on ROCm).  The reference's setter
    assigns a local and never takes effect; this one does."""
    _STATE["trace"] = bool(flag)


def get_nvtx():
    return _STATE["trace"]
