# The edit the reference's generic residency code needs before a ROCm backend can attach a
# resident arena or a workspace: src/backend/residency.c:32 and :206 admit the CUDA kind only.
# Applied on the fly while that file is compiled from where it lies (oracle/Makefile, target
# ref_backend); the same edit is listed for maintainers in INTEGRATION.md.
/^int yvex_backend_resident_attach/,/^}/ s/backend->kind != YVEX_BACKEND_KIND_CUDA ||/(backend->kind != YVEX_BACKEND_KIND_CUDA \&\& backend->kind != YVEX_BACKEND_KIND_ROCM) ||/
/^int yvex_backend_workspace_attach/,/^}/ s/backend->kind != YVEX_BACKEND_KIND_CUDA ||/(backend->kind != YVEX_BACKEND_KIND_CUDA \&\& backend->kind != YVEX_BACKEND_KIND_ROCM) ||/
