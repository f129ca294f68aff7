classdef DeviceSet < handle
    % Owner of one device-resident set handle of libnnvhip.so.  MATLAB copies of a Star value share
    % this handle object; the device memory is released when the last copy goes away.
    properties (SetAccess = private)
        h uint64 = uint64(0);   % opaque nnvhip_star* from the MEX gateway
    end
    methods
        function obj = DeviceSet(h)
            obj.h = h;
        end
        function delete(obj)
            if obj.h ~= 0
                nnvhip_mex('star_release', obj.h);
                obj.h = uint64(0);
            end
        end
    end
end
