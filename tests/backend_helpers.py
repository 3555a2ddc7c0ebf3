"""The backend conveniences the contract tests share live in the package."""
from yvex_amd.host import Backend  # noqa: F401
