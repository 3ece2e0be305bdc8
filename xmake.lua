-- xmake build of libinfiniop.so with the amd-gpu device (AMD Instinct MI355X, gfx950 only).
--
--     xmake f --amd-gpu=y && xmake && xmake install      -- into $INFINI_ROOT (default ~/.infini)
--
-- Same targets and install layout as the reference's xmake.lua (reference
-- xmake.lua:9-41 options, :69-107 a GPU back end as a static target, :215-238
-- the shared target "infiniop" installed under $INFINI_ROOT/{lib,include}),
-- for this repository's source tree.  xmake is not part of the image this
-- library is developed in, so this file is NOT exercised there: the build that
-- is exercised, with the same compiler and flags, is
-- `python -m operators_amd.build [--install]`.
add_rules("mode.debug", "mode.release")
add_includedirs("include")

option("amd-gpu")
    set_default(true)
    set_showmenu(true)
    set_description("Enable or disable the AMD Instinct MI355X (gfx950) kernels")
    add_defines("ENABLE_AMD_GPU")
option_end()

local ROCM = os.getenv("ROCM_PATH") or "/opt/rocm"
local HIPCC = ROCM .. "/bin/hipcc"
local CSRC = "operators_amd/csrc"

-- One offload architecture, no CUDA headers, no second code path.
--   -ffp-contract=off : RoPE's products round before the add that follows them, as on the reference's CPU
--   -packed-fp32-ops  : no packed fp32 instructions from auto-vectorisation
local HIP_FLAGS = {
    "-std=c++17", "-O3", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off",
    "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
}

if has_config("amd-gpu") then

    add_defines("ENABLE_AMD_GPU")

    -- .hip and .cc files of the back end both go through hipcc: the host-only
    -- files still need the HIP runtime headers.
    rule("hipcc")
        set_extensions(".hip", ".cc")
        on_build_file(function (target, sourcefile)
            local objectfile = target:objectfile(sourcefile)
            os.mkdir(path.directory(objectfile))
            local args = {}
            for _, flag in ipairs(HIP_FLAGS) do
                table.insert(args, flag)
            end
            if sourcefile:endswith(".cc") then
                table.insert(args, "-x")
                table.insert(args, "c++")
                table.insert(args, "-D__HIP_PLATFORM_AMD__")
                table.insert(args, "-I" .. ROCM .. "/include")
            end
            for _, dir in ipairs(target:get("includedirs")) do
                table.insert(args, "-I" .. dir)
            end
            table.insert(args, "-c")
            table.insert(args, sourcefile)
            table.insert(args, "-o")
            table.insert(args, objectfile)
            os.execv(HIPCC, args)
            table.insert(target:objectfiles(), objectfile)
        end)
    rule_end()

    target("amd-gpu")
        set_kind("static")
        on_install(function (target) end)
        set_languages("cxx17")
        add_includedirs("include")
        -- only the hipcc rule compiles this target's files: `rules = ` replaces the rules xmake would pick by
        -- extension (for .cc its own C++ rule, which would compile every file a second time)
        add_files(CSRC .. "/devices/amd/*.cc", {rules = "hipcc"})
        add_files(CSRC .. "/ops/*/amd/*.cc", {rules = "hipcc"})
        add_files(CSRC .. "/ops/*/amd/*.hip", {rules = "hipcc"})
    target_end()

end

target("infiniop")
    set_kind("shared")
    if has_config("amd-gpu") then
        add_deps("amd-gpu")
    end
    set_languages("cxx17")
    set_toolset("ld", HIPCC)
    set_toolset("sh", HIPCC)
    add_shflags("--offload-arch=gfx950", {force = true})
    add_syslinks("dl", "pthread")   -- the BLAS loader calls dlopen / dlsym; glibc before 2.34 keeps them in libdl
    add_includedirs(ROCM .. "/include")
    add_defines("__HIP_PLATFORM_AMD__")
    add_cxxflags("-fPIC", "-fvisibility=hidden")
    add_files(CSRC .. "/devices/handle.cc")
    add_files(CSRC .. "/ops/*/operator.cc")
    add_files(CSRC .. "/tensor/*.cc")

    set_installdir(os.getenv("INFINI_ROOT") or (os.getenv("HOME") .. "/.infini"))
    add_installfiles("include/(**/*.h)", {prefixdir = "include"})
    add_installfiles("include/*.h", {prefixdir = "include"})
target_end()
